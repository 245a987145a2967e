"""GPU tests of the per-token writers (fused QK-Norm + RoPE + K/V append, sin/cos table, cache re-stride),
of the pooled device allocator, and of the captured multi-layer decode stack, against the CPU oracle."""
import ctypes
import os

import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import assert_parity, from_dev_bf16, to_dev

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bf16_close(got_bits, want_bits, what):
    """Outputs of the fused norm/rope chain: at most one bf16 ulp apart, and almost all identical. The
    reference's own tolerance for this op is atol = rtol = 2e-2 (test_qwen3_bf16_ops.py:836-917)."""
    g = synth.bf16_bits_to_f32(got_bits).astype(np.float64)
    w = synth.bf16_bits_to_f32(want_bits).astype(np.float64)
    assert np.all(np.abs(g - w) <= np.abs(w) / 128 + 1e-6), what
    assert (got_bits == want_bits).mean() > 0.99, what


def test_sincos_table_matches_oracle(oracle, dev):
    sin_d, cos_d = ops.sincos_table(128, 5000, dev)
    torch.cuda.synchronize()
    sin_o, cos_o = oracle.sincos_table(128, 5000)
    # the reference's own tolerance for this table is 2e-6 (test_qwen3_bf16_ops.py:857-858)
    assert np.abs(sin_d.cpu().numpy() - sin_o).max() <= 2e-6
    assert np.abs(cos_d.cpu().numpy() - cos_o).max() <= 2e-6


@pytest.mark.parametrize("layout", [B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])
@pytest.mark.parametrize("n_q,n_kv", [(32, 8), (64, 8), (16, 8)])
def test_qk_norm_rope_append(oracle, dev, layout, n_q, n_kv):
    rng = np.random.RandomState(n_q + layout)
    d, layers, msl, layer_id, pos = 128, 3, 50, 2, 41
    kv_dim = n_kv * d
    q = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
    k_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    v_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    sin_o, cos_o = oracle.sincos_table(d, msl)
    q_ref = oracle.qk_norm_rope(q, w[:d], sin_o[pos], cos_o[pos])
    k_ref = oracle.qk_norm_rope(k_new, w[d:], sin_o[pos], cos_o[pos])

    cache_shape = (layers, msl, kv_dim) if layout == 0 else (layers, n_kv, msl, d)
    k_cache = torch.full(cache_shape, 0x1234, dtype=torch.int16, device=dev)
    v_cache = torch.full(cache_shape, 0x1234, dtype=torch.int16, device=dev)
    q_d = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    ops.qk_norm_rope_append(q_d, to_dev(k_new.reshape(-1), dev), to_dev(v_new.reshape(-1), dev), k_cache, v_cache,
                            to_dev(w, dev), sin_d, cos_d, layer_id=layer_id, pos=pos, kv_dim=kv_dim, head_num=n_q,
                            head_dim=d, max_seq_len=msl, kv_layout=layout, query_src=to_dev(q.reshape(-1), dev))
    torch.cuda.synchronize()
    _bf16_close(q_d.cpu().numpy().view(np.uint16).reshape(n_q, d), q_ref, "query")
    kc = k_cache.cpu().numpy().view(np.uint16)
    vc = v_cache.cpu().numpy().view(np.uint16)
    if layout == 0:
        k_row, v_row = kc[layer_id, pos].reshape(n_kv, d).copy(), vc[layer_id, pos].reshape(n_kv, d).copy()
        kc[layer_id, pos] = 0x1234
        vc[layer_id, pos] = 0x1234
    else:
        k_row, v_row = kc[layer_id, :, pos].copy(), vc[layer_id, :, pos].copy()
        kc[layer_id, :, pos] = 0x1234
        vc[layer_id, :, pos] = 0x1234
    _bf16_close(k_row, k_ref, "key row")
    assert np.array_equal(v_row, v_new)                    # V is copied bit for bit
    assert np.all(kc == 0x1234) and np.all(vc == 0x1234)  # nothing else in the caches was touched


def test_qk_norm_rope_in_place_on_the_cache_row(oracle, dev):
    """The reference's call pattern: K row already in its position-major cache slot, transformed in place,
    V untouched (rmsnorm_kernel.cu:248-290 with model.cpp:90-107)."""
    rng = np.random.RandomState(3)
    d, n_q, n_kv, msl, pos = 128, 32, 8, 16, 9
    q = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
    cache = synth.f32_to_bf16_bits(rng.standard_normal((1, msl, n_kv * d)).astype(np.float32))
    w = synth.f32_to_bf16_bits(np.ones(2 * d, dtype=np.float32))
    sin_o, cos_o = oracle.sincos_table(d, msl)
    k_ref = oracle.qk_norm_rope(cache[0, pos].reshape(n_kv, d), w[d:], sin_o[pos], cos_o[pos])
    q_ref = oracle.qk_norm_rope(q, w[:d], sin_o[pos], cos_o[pos])
    k_cache = to_dev(cache, dev)
    q_d = to_dev(q.reshape(-1), dev)
    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    row = k_cache[0, pos]  # contiguous view of the slot
    ops.qk_norm_rope_append(q_d, row, None, k_cache, None, to_dev(w, dev), sin_d, cos_d, layer_id=0, pos=pos,
                            kv_dim=n_kv * d, head_num=n_q, head_dim=d, max_seq_len=msl)
    torch.cuda.synchronize()
    got = k_cache.cpu().numpy().view(np.uint16)
    _bf16_close(got[0, pos].reshape(n_kv, d), k_ref, "key row")
    _bf16_close(q_d.cpu().numpy().view(np.uint16).reshape(n_q, d), q_ref, "query")
    mask = np.ones(msl, dtype=bool)
    mask[pos] = False
    assert np.array_equal(got[0, mask], cache[0, mask])


def test_kv_restride_is_a_permutation(dev):
    layers, msl, n_kv, d, num_pos = 3, 37, 8, 128, 30
    src = np.random.RandomState(0).randint(0, 65536, size=(layers, msl, n_kv * d)).astype(np.uint16)
    dst = torch.zeros((layers, n_kv, msl, d), dtype=torch.int16, device=dev)
    ops.kv_restride(to_dev(src, dev), dst, layer_num=layers, max_seq_len=msl, kv_dim=n_kv * d, head_dim=d,
                    num_pos=num_pos)
    torch.cuda.synchronize()
    got = dst.cpu().numpy().view(np.uint16)
    want = synth.to_head_major(src, n_kv)
    assert np.array_equal(got[:, :, :num_pos], want[:, :, :num_pos])
    assert not got[:, :, num_pos:].any()  # rows past num_pos are left alone


def test_attention_after_append_uses_the_new_row(oracle, dev):
    """Append token `pos` with the fused kernel, then attend over 0..pos: equals the oracle run on a cache
    whose row `pos` holds the oracle's normalised K row and the raw V row."""
    rng = np.random.RandomState(8)
    n_q, n_kv, d, ctx = 32, 8, 128, 600
    case = synth.make_case(55, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=ctx + 1)
    pos = ctx
    q_raw = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
    k_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    v_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    sin_o, cos_o = oracle.sincos_table(d, ctx + 1)
    q_n = oracle.qk_norm_rope(q_raw, w[:d], sin_o[pos], cos_o[pos])
    k_ref, v_ref = case["k"].copy(), case["v"].copy()
    k_ref[0, pos] = oracle.qk_norm_rope(k_new, w[d:], sin_o[pos], cos_o[pos]).reshape(-1)
    v_ref[0, pos] = v_new.reshape(-1)
    ref = oracle.mha_cpu(q_n.reshape(-1), k_ref, v_ref, 0, pos, n_kv * d, n_q // n_kv, n_q, d, ctx + 1)

    k_d = to_dev(synth.to_head_major(case["k"], n_kv), dev)
    v_d = to_dev(synth.to_head_major(case["v"], n_kv), dev)
    q_d = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    out = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    ws = torch.empty(ops.workspace_bytes(n_q, d, ctx + 1) // 4, dtype=torch.float32, device=dev)
    sin_d, cos_d = ops.sincos_table(d, ctx + 1, dev)
    kw = dict(layer_id=0, pos=pos, kv_dim=n_kv * d, head_num=n_q, head_dim=d, max_seq_len=ctx + 1,
              kv_layout=B.KV_LAYOUT_HEAD_MAJOR)
    ops.qk_norm_rope_append(q_d, to_dev(k_new.reshape(-1), dev), to_dev(v_new.reshape(-1), dev), k_d, v_d,
                            to_dev(w, dev), sin_d, cos_d, query_src=to_dev(q_raw.reshape(-1), dev), **kw)
    ops.mha_decode(q_d, k_d, v_d, out, ws, kv_mul=n_q // n_kv, **kw)
    torch.cuda.synchronize()
    assert_parity(from_dev_bf16(out), ref, "append + attention")


@pytest.mark.parametrize("layout", [B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])
@pytest.mark.parametrize("n_q,n_kv,ctx,path,splits", [
    (32, 8, 600, B.PATH_AUTO, 0), (32, 8, 4096, B.PATH_AUTO, 0), (32, 8, 100, B.PATH_AUTO, 0),
    (32, 8, 0, B.PATH_AUTO, 0), (32, 8, 15, B.PATH_SINGLE_PASS, 0), (32, 8, 16, B.PATH_SINGLE_PASS, 0),
    (32, 8, 1023, B.PATH_SPLIT_FUSED, 7), (32, 8, 1024, B.PATH_SPLIT_FUSED, 64), (64, 8, 777, B.PATH_AUTO, 0),
    (16, 8, 300, B.PATH_AUTO, 0), (12, 4, 333, B.PATH_SPLIT_FUSED, 5),
    # groups of 8 query heads run 8 waves per workgroup, like the plain kernel (Qwen3-32B head layout)
    (64, 8, 4096, B.PATH_AUTO, 0), (64, 8, 32768, B.PATH_AUTO, 0), (64, 8, 131072, B.PATH_AUTO, 0),
])
def test_fused_append_attention(oracle, dev, layout, n_q, n_kv, ctx, path, splits):
    """llmi_hip_mha_decode_append (norm + rope + append + attention in one launch) against the oracle chain:
    normalise q and the new K row, put K/V at `pos`, attend over 0..pos; the cache rows it must have written
    are checked too, and nothing else in the caches may change. ctx = cached positions before the new token."""
    rng = np.random.RandomState(ctx + n_q)
    d, msl, pos, kv_dim = 128, ctx + 3, ctx, n_kv * 128
    case = synth.make_case(500 + ctx, n_q=n_q, n_kv=n_kv, ctx=max(ctx, 1), max_seq_len=msl)
    k0, v0 = case["k"].copy(), case["v"].copy()
    k0[0, ctx:] = 0x7FC0  # rows from the new position on are NaN patterns until written
    v0[0, ctx:] = 0x7FC0
    q_raw = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
    k_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    v_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    sin_o, cos_o = oracle.sincos_table(d, msl)
    q_n = oracle.qk_norm_rope(q_raw, w[:d], sin_o[pos], cos_o[pos])
    k_n = oracle.qk_norm_rope(k_new, w[d:], sin_o[pos], cos_o[pos])
    k_ref, v_ref = k0.copy(), v0.copy()
    k_ref[0, pos] = k_n.reshape(-1)
    v_ref[0, pos] = v_new.reshape(-1)
    ref = oracle.mha_cpu(q_n.reshape(-1), k_ref, v_ref, 0, pos, kv_dim, n_q // n_kv, n_q, d, msl)

    hm = layout == B.KV_LAYOUT_HEAD_MAJOR
    k_d = to_dev(synth.to_head_major(k0, n_kv) if hm else k0, dev)
    v_d = to_dev(synth.to_head_major(v0, n_kv) if hm else v0, dev)
    out = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    ws = torch.full((ops.workspace_bytes(n_q, d, msl) // 4,), float("nan"), dtype=torch.float32, device=dev)
    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    ops.mha_decode_append(to_dev(q_raw.reshape(-1), dev), to_dev(k_new.reshape(-1), dev),
                          to_dev(v_new.reshape(-1), dev), to_dev(w, dev), sin_d, cos_d, k_d, v_d, out, ws,
                          layer_id=0, pos=pos, kv_dim=kv_dim, kv_mul=n_q // n_kv, head_num=n_q, head_dim=d,
                          max_seq_len=msl, kv_layout=layout, force_path=path, num_splits=splits)
    torch.cuda.synchronize()
    assert_parity(from_dev_bf16(out), ref, "fused append ctx=%d" % ctx)
    kc = k_d.cpu().numpy().view(np.uint16)
    vc = v_d.cpu().numpy().view(np.uint16)
    if hm:
        kc = np.ascontiguousarray(kc.transpose(0, 2, 1, 3)).reshape(1, msl, kv_dim)
        vc = np.ascontiguousarray(vc.transpose(0, 2, 1, 3)).reshape(1, msl, kv_dim)
    _bf16_close(kc[0, pos].reshape(n_kv, d), k_n, "appended key row")
    assert np.array_equal(vc[0, pos], v_new.reshape(-1))
    keep = np.ones(msl, dtype=bool)
    keep[pos] = False
    assert np.array_equal(kc[0, keep], k0[0, keep]) and np.array_equal(vc[0, keep], v0[0, keep])
    if ctx <= 4096:
        # the same call with the workspace laid out by package side (measured, then the opposite claim): same bits
        measured = ops.workspace_side(ws)
        for side in (measured, 0x55555555 if measured & 2 else -1431655766):
            k2 = to_dev(synth.to_head_major(k0, n_kv) if hm else k0, dev)
            v2 = to_dev(synth.to_head_major(v0, n_kv) if hm else v0, dev)
            out2 = torch.zeros_like(out)
            ops.mha_decode_append(to_dev(q_raw.reshape(-1), dev), to_dev(k_new.reshape(-1), dev),
                                  to_dev(v_new.reshape(-1), dev), to_dev(w, dev), sin_d, cos_d, k2, v2, out2, ws,
                                  layer_id=0, pos=pos, kv_dim=kv_dim, kv_mul=n_q // n_kv, head_num=n_q, head_dim=d,
                                  max_seq_len=msl, kv_layout=layout, force_path=path, num_splits=splits, workspace_side=side)
            torch.cuda.synchronize()
            assert torch.equal(out2, out) and torch.equal(k2, k_d) and torch.equal(v2, v_d), "workspace_side %x" % (side & 0xFFFFFFFF)


def test_default_pool_on_device(dev):
    lib = B.lib()
    a = lib.llmi_hip_pool_alloc(4)
    assert a and lib.llmi_hip_pool_free(a) == 0
    assert lib.llmi_hip_pool_alloc(4) == a
    big = lib.llmi_hip_pool_alloc(5 << 20)
    assert big and lib.llmi_hip_memset_zero(big, 5 << 20, None, 1) == 0
    host = (ctypes.c_uint8 * 16)(*range(16))
    back = (ctypes.c_uint8 * 16)()
    assert lib.llmi_hip_memcpy(big, host, 16, 1, None, 1) == 0
    assert lib.llmi_hip_memcpy(back, big, 16, 2, None, 1) == 0
    assert list(back) == list(range(16))
    assert lib.llmi_hip_pool_free(big) == 0 and lib.llmi_hip_pool_free(big) == B.STATUS["UNKNOWN_POINTER"]
    assert lib.llmi_hip_pool_alloc((5 << 20) - 4096) == big


# ---------------------------------------------------------------- the captured multi-layer stack
class HostLib:
    def __init__(self):
        L = ctypes.CDLL(os.path.join(ROOT, "llminfer_amd", "libllmi_host.so"))
        L.llmi_host_stack_create.restype = ctypes.c_void_p
        L.llmi_host_stack_create.argtypes = [ctypes.c_int32] * 5
        L.llmi_host_stack_destroy.argtypes = [ctypes.c_void_p]
        L.llmi_host_stack_ptr.restype = ctypes.c_void_p
        L.llmi_host_stack_ptr.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
        for name in ("llmi_host_stack_build_sincos",):
            getattr(L, name).argtypes = [ctypes.c_void_p]
        L.llmi_host_stack_run.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
        L.llmi_host_stack_capture.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
        L.llmi_host_stack_replay.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_float)]
        L.llmi_host_last_error.restype = ctypes.c_char_p
        L.llmi_host_mha_forward.argtypes = ([ctypes.c_void_p] * 4 + [ctypes.c_int64, ctypes.c_void_p] +
                                            [ctypes.c_int32] * 9)
        self.L = L

    def ok(self, rc):
        assert rc == 0, self.L.llmi_host_last_error().decode()


def _upload(ptr, arr):
    arr = np.ascontiguousarray(arr)
    rc = B.lib().llmi_hip_memcpy(ptr, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes, 1, None, 1)
    assert rc == 0


def _download(ptr, shape, dtype):
    out = np.empty(shape, dtype=dtype)
    assert B.lib().llmi_hip_memcpy(out.ctypes.data_as(ctypes.c_void_p), ptr, out.nbytes, 2, None, 1) == 0
    return out


@pytest.mark.parametrize("layout,layers,ctx", [(B.KV_LAYOUT_POS_MAJOR, 4, 300), (B.KV_LAYOUT_HEAD_MAJOR, 4, 300),
                                               (B.KV_LAYOUT_HEAD_MAJOR, 36, 4096)])
def test_decode_stack_eager_and_graph_match_oracle(oracle, dev, layout, layers, ctx):
    """Layers of (QK-Norm + RoPE + append, attention) at ctx + 1 new token: eager run and several replays
    of the captured graph all match the oracle layer by layer. 4 layers at ctx 300 in both layouts, and the
    Qwen3-4B stack at its full size: 36 layers at ctx 4096, 36 independently seeded per-layer caches."""
    H = HostLib()
    n_q, n_kv, d = 32, 8, 128
    msl, pos, kv_dim = ctx + 1, ctx, n_kv * d
    stack = H.L.llmi_host_stack_create(layers, msl, n_q, n_kv, layout)
    assert stack, H.L.llmi_host_last_error().decode()
    try:
        H.ok(H.L.llmi_host_stack_build_sincos(stack))
        rng = np.random.RandomState(4)
        k_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        v_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        raw = []
        for l in range(layers):  # every layer its own seeded cache
            c = synth.make_case(400 + l, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
            k_all[l], v_all[l] = c["k"][0], c["v"][0]
            qr = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
            kr = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
            vr = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
            w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
            raw.append((qr, kr, vr, w))
            for which, arr in ((2, qr), (3, kr), (4, vr), (5, w)):
                _upload(H.L.llmi_host_stack_ptr(stack, which, l), arr)
        k_up = k_all if layout == 0 else synth.to_head_major(k_all, n_kv)
        v_up = v_all if layout == 0 else synth.to_head_major(v_all, n_kv)
        _upload(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up)
        _upload(H.L.llmi_host_stack_ptr(stack, 1, 0), v_up)

        sin_o, cos_o = oracle.sincos_table(d, msl)
        refs = []
        for l in range(layers):
            qr, kr, vr, w = raw[l]
            k_ref, v_ref = k_all[l:l + 1].copy(), v_all[l:l + 1].copy()
            k_ref[0, pos] = oracle.qk_norm_rope(kr, w[d:], sin_o[pos], cos_o[pos]).reshape(-1)
            v_ref[0, pos] = vr.reshape(-1)
            qn = oracle.qk_norm_rope(qr, w[:d], sin_o[pos], cos_o[pos]).reshape(-1)
            refs.append(oracle.mha_cpu(qn, k_ref, v_ref, 0, pos, kv_dim, n_q // n_kv, n_q, d, msl))

        def check(tag):
            for l in range(layers):
                got = _download(H.L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,), np.uint16)
                assert_parity(synth.bf16_bits_to_f32(got), refs[l], "%s layer %d" % (tag, l))

        H.ok(H.L.llmi_host_stack_run(stack, pos, 1))
        check("eager")
        k_after = _download(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up.shape, np.uint16)
        _upload(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up)  # forget the appended rows
        _upload(H.L.llmi_host_stack_ptr(stack, 1, 0), v_up)
        for l in range(layers):
            _upload(H.L.llmi_host_stack_ptr(stack, 6, l), np.zeros(n_q * d, dtype=np.uint16))
        H.ok(H.L.llmi_host_stack_run(stack, pos, 2))  # the same step with norm/rope/append fused into attention
        check("eager fused append")
        k_fused = _download(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up.shape, np.uint16)
        assert (k_fused == k_after).mean() > 0.9999  # the appended K rows agree up to rare bf16 rounding flips
        H.ok(H.L.llmi_host_stack_capture(stack, pos, 2))
        ms = ctypes.c_float()
        for rep in range(3):
            for l in range(layers):  # wipe the outputs between replays
                _upload(H.L.llmi_host_stack_ptr(stack, 6, l), np.zeros(n_q * d, dtype=np.uint16))
            H.ok(H.L.llmi_host_stack_replay(stack, 1, ctypes.byref(ms)))
            check("replay %d" % rep)
            torch.randn(1000, device=dev).sum().item()  # eager work between replays
        assert ms.value > 0
        # the same step as ONE resident launch for all layers (mode 5): the bits of mode 2, eager and replayed
        want = [_download(H.L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,), np.uint16) for l in range(layers)]

        def check_bits(tag):
            for l in range(layers):
                got = _download(H.L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,), np.uint16)
                assert np.array_equal(got, want[l]), "%s layer %d" % (tag, l)

        def wipe():
            _upload(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up)
            _upload(H.L.llmi_host_stack_ptr(stack, 1, 0), v_up)
            for l in range(layers):
                _upload(H.L.llmi_host_stack_ptr(stack, 6, l), np.zeros(n_q * d, dtype=np.uint16))

        wipe()
        H.ok(H.L.llmi_host_stack_run(stack, pos, 5))
        check_bits("resident, eager")
        assert np.array_equal(_download(H.L.llmi_host_stack_ptr(stack, 0, 0), k_up.shape, np.uint16), k_fused)
        H.ok(H.L.llmi_host_stack_capture(stack, pos, 5))
        for rep in range(3):
            wipe()
            H.ok(H.L.llmi_host_stack_replay(stack, 1, ctypes.byref(ms)))
            check_bits("resident, replay %d" % rep)
            torch.randn(1000, device=dev).sum().item()
    finally:
        H.L.llmi_host_stack_destroy(stack)


def test_decode_stack_graph_follows_the_device_position(oracle, dev):
    """One captured 3-layer stack (norm/rope/append fused into attention) decodes four successive tokens:
    only the raw inputs and the position word change between replays."""
    H = HostLib()
    H.L.llmi_host_stack_capture_following.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    H.L.llmi_host_stack_set_pos.argtypes = [ctypes.c_void_p, ctypes.c_int32]
    layers, ctx, n_q, n_kv, d, tokens, layout = 3, 270, 32, 8, 128, 4, B.KV_LAYOUT_HEAD_MAJOR
    msl, kv_dim = ctx + tokens, n_kv * d
    stack = H.L.llmi_host_stack_create(layers, msl, n_q, n_kv, layout)
    assert stack, H.L.llmi_host_last_error().decode()
    try:
        H.ok(H.L.llmi_host_stack_build_sincos(stack))
        rng = np.random.RandomState(14)
        k_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        v_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        ws = []
        for l in range(layers):
            c = synth.make_case(700 + l, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
            k_all[l], v_all[l] = c["k"][0], c["v"][0]
            w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
            ws.append(w)
            _upload(H.L.llmi_host_stack_ptr(stack, 5, l), w)
        _upload(H.L.llmi_host_stack_ptr(stack, 0, 0), synth.to_head_major(k_all, n_kv))
        _upload(H.L.llmi_host_stack_ptr(stack, 1, 0), synth.to_head_major(v_all, n_kv))
        sin_o, cos_o = oracle.sincos_table(d, msl)
        H.ok(H.L.llmi_host_stack_set_pos(stack, ctx))
        H.ok(H.L.llmi_host_stack_capture_following(stack, msl - 1, 2))
        ms = ctypes.c_float()
        for pos in range(ctx, ctx + tokens):
            refs = []
            for l in range(layers):
                qr = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
                kr = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
                vr = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
                for which, arr in ((2, qr), (3, kr), (4, vr)):
                    _upload(H.L.llmi_host_stack_ptr(stack, which, l), arr)
                k_all[l, pos] = oracle.qk_norm_rope(kr, ws[l][d:], sin_o[pos], cos_o[pos]).reshape(-1)
                v_all[l, pos] = vr.reshape(-1)
                qn = oracle.qk_norm_rope(qr, ws[l][:d], sin_o[pos], cos_o[pos]).reshape(-1)
                refs.append(oracle.mha_cpu(qn, k_all[l:l + 1], v_all[l:l + 1], 0, pos, kv_dim, n_q // n_kv, n_q, d, msl))
            H.ok(H.L.llmi_host_stack_set_pos(stack, pos))
            H.ok(H.L.llmi_host_stack_replay(stack, 1, ctypes.byref(ms)))
            for l in range(layers):
                got = _download(H.L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,), np.uint16)
                assert_parity(synth.bf16_bits_to_f32(got), refs[l], "token at %d, layer %d" % (pos, l))
    finally:
        H.L.llmi_host_stack_destroy(stack)


@pytest.mark.parametrize("mode", [3, 4])
def test_attention_block_stack_matches_the_oracle_chain(oracle, dev, mode):
    """Modes 3 and 4 of the stack, two layers: packed QKV GEMV -> QK-Norm + RoPE + append + attention -> output
    projection added to the residual stream (mode 4: attention and projection in one launch). The oracle
    replays the chain with a bf16 rounding wherever the kernels store bf16 (GEMV outputs, attention
    output, residual)."""
    H = HostLib()
    H.L.llmi_host_stack_enable_projections.argtypes = [ctypes.c_void_p, ctypes.c_int32]
    layers, ctx, n_q, n_kv, d, hidden, layout = 2, 280, 16, 8, 128, 1024, B.KV_LAYOUT_HEAD_MAJOR
    dim, kv_dim, msl, pos = n_q * d, n_kv * d, ctx + 1, ctx
    stack = H.L.llmi_host_stack_create(layers, msl, n_q, n_kv, layout)
    assert stack, H.L.llmi_host_last_error().decode()
    try:
        H.ok(H.L.llmi_host_stack_enable_projections(stack, hidden))
        H.ok(H.L.llmi_host_stack_build_sincos(stack))
        rng = np.random.RandomState(21)
        sin_o, cos_o = oracle.sincos_table(d, msl)
        k_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        v_all = np.zeros((layers, msl, kv_dim), dtype=np.uint16)
        res0 = synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32))
        res_ref = synth.bf16_bits_to_f32(res0).copy()
        attn_refs = []
        for l in range(layers):
            c = synth.make_case(800 + l, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
            k_all[l], v_all[l] = c["k"][0], c["v"][0]
            x = synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32))
            wqkv = synth.f32_to_bf16_bits((rng.standard_normal((dim + 2 * kv_dim, hidden)) / np.sqrt(hidden)).astype(np.float32))
            wo = synth.f32_to_bf16_bits((rng.standard_normal((hidden, dim)) / np.sqrt(dim)).astype(np.float32))
            w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
            for which, arr in ((12, x), (10, wqkv), (11, wo), (5, w)):
                _upload(H.L.llmi_host_stack_ptr(stack, which, l), arr)
            qkv = synth.f32_to_bf16_bits(oracle.gemv_bf16(x, wqkv))
            qr, kr, vr = qkv[:dim].reshape(n_q, d), qkv[dim:dim + kv_dim].reshape(n_kv, d), qkv[dim + kv_dim:]
            k_all[l, pos] = oracle.qk_norm_rope(kr, w[d:], sin_o[pos], cos_o[pos]).reshape(-1)
            v_all[l, pos] = vr
            qn = oracle.qk_norm_rope(qr, w[:d], sin_o[pos], cos_o[pos]).reshape(-1)
            attn = oracle.mha_cpu(qn, k_all[l:l + 1], v_all[l:l + 1], 0, pos, kv_dim, n_q // n_kv, n_q, d, msl)
            attn_refs.append(attn)
            proj = oracle.gemv_bf16(synth.f32_to_bf16_bits(attn), wo)
            res_ref = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(res_ref + proj))
        k_up = k_all.copy()
        v_up = v_all.copy()
        k_up[:, pos], v_up[:, pos] = 0x7FC0, 0x7FC0  # the new rows are the kernels' to write
        _upload(H.L.llmi_host_stack_ptr(stack, 0, 0), synth.to_head_major(k_up, n_kv))
        _upload(H.L.llmi_host_stack_ptr(stack, 1, 0), synth.to_head_major(v_up, n_kv))
        _upload(H.L.llmi_host_stack_ptr(stack, 13, 0), res0)
        H.ok(H.L.llmi_host_stack_run(stack, pos, mode))
        for l in range(layers):
            got = _download(H.L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,), np.uint16)
            assert_parity(synth.bf16_bits_to_f32(got), attn_refs[l], "block layer %d attention" % l)
        res = synth.bf16_bits_to_f32(_download(H.L.llmi_host_stack_ptr(stack, 13, 0), (hidden,), np.uint16))
        # residual of magnitude ~1: one bf16 step is 2^-8 relative; the projections add O(1) values
        assert np.all(np.abs(res - res_ref) <= np.abs(res_ref) / 64 + 2e-2), np.abs(res - res_ref).max()
        # graph replay of the block gives the same residual increment again
        _upload(H.L.llmi_host_stack_ptr(stack, 13, 0), res0)
        H.ok(H.L.llmi_host_stack_capture(stack, pos, mode))
        ms = ctypes.c_float()
        for rep in range(3):  # replays of one graph: the per-head counters of the fused projection keep moving
            _upload(H.L.llmi_host_stack_ptr(stack, 13, 0), res0)
            H.ok(H.L.llmi_host_stack_replay(stack, 1, ctypes.byref(ms)))
            res2 = synth.bf16_bits_to_f32(_download(H.L.llmi_host_stack_ptr(stack, 13, 0), (hidden,), np.uint16))
            assert np.array_equal(res, res2), "replay %d" % rep
            torch.randn(1000, device=dev).sum().item()  # eager work between replays
    finally:
        H.L.llmi_host_stack_destroy(stack)


@pytest.mark.parametrize("n_q,ctx,hidden,want_launches,extra", [
    (32, 4096, 2560, 1, {}),      # Qwen3-4B: 32 splits, 248 worker workgroups, rows dealt 3 / 3 / 2 per wavefront
    (32, 4096, 2560, 1, {"num_splits": 32, "force_path": B.PATH_SPLIT_FUSED}),  # the same plan in both forms: same bits
    (32, 8192, 2560, 1, {}),
    (32, 3500, 2560, 1, {}),
    (32, 1500, 2560, 1, {}),      # (the dispatcher would take 16 splits here: the one-launch form asks for 32 itself)
    (16, 700, 1024, 1, {}),       # Qwen3-0.6B head layout
    (64, 5000, 640, 2, {}),       # attention output wider than the fused form takes: two launches, same answer
    (32, 100, 2560, 2, {}),       # single pass: nothing idles, two launches
    (32, 4096, 2560, 2, {"num_splits": 2, "force_path": B.PATH_SPLIT_FUSED}),  # too few workers for 2560 rows
])
def test_fused_output_projection_equals_attention_then_gemv_add(oracle, dev, n_q, ctx, hidden, want_launches, extra):
    """llmi_hip_mha_decode_append_oproj against llmi_hip_mha_decode_append followed by llmi_hip_gemv (add mode) on
    the same inputs: same attention output and same residual bit for bit where both forms run the same plan; the
    attention output also against the oracle. Called three times in a row on one workspace (its per-head counters move on)."""
    n_kv, d = 8, 128
    rng = np.random.RandomState(ctx + hidden)
    msl, pos, kv_dim, dim = ctx + 2, ctx, n_kv * d, n_q * d
    case = synth.make_case(900 + ctx, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
    k0, v0 = case["k"].copy(), case["v"].copy()
    q_raw = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
    k_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    v_new = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    wo = synth.f32_to_bf16_bits((rng.standard_normal((hidden, dim)) / np.sqrt(dim)).astype(np.float32))
    res0 = synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32))
    sin_o, cos_o = oracle.sincos_table(d, msl)
    k_ref, v_ref = k0.copy(), v0.copy()
    k_ref[0, pos] = oracle.qk_norm_rope(k_new, w[d:], sin_o[pos], cos_o[pos]).reshape(-1)
    v_ref[0, pos] = v_new.reshape(-1)
    q_n = oracle.qk_norm_rope(q_raw, w[:d], sin_o[pos], cos_o[pos])
    ref = oracle.mha_cpu(q_n.reshape(-1), k_ref, v_ref, 0, pos, kv_dim, n_q // n_kv, n_q, d, msl)

    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    wo_d, w_d = to_dev(wo.reshape(-1), dev), to_dev(w, dev)
    qd, kd, vd = to_dev(q_raw.reshape(-1), dev), to_dev(k_new.reshape(-1), dev), to_dev(v_new.reshape(-1), dev)
    ws = torch.full((ops.workspace_bytes(n_q, d, msl) // 4,), float("nan"), dtype=torch.float32, device=dev)
    kw = dict(layer_id=0, pos=pos, kv_dim=kv_dim, kv_mul=n_q // n_kv, head_num=n_q, head_dim=d, max_seq_len=msl,
              kv_layout=B.KV_LAYOUT_HEAD_MAJOR, **extra)

    def fresh():
        return (to_dev(synth.to_head_major(k0, n_kv), dev), to_dev(synth.to_head_major(v0, n_kv), dev),
                torch.zeros(dim, dtype=torch.int16, device=dev), to_dev(res0, dev))

    # the two-call form
    kc, vc, out_a, res_a = fresh()
    ops.mha_decode_append(qd, kd, vd, w_d, sin_d, cos_d, kc, vc, out_a, ws, **kw)
    ops.gemv(out_a, wo_d.view(hidden, dim), res_a, mode=B.GEMV_ADD_BF16)
    torch.cuda.synchronize()
    assert_parity(from_dev_bf16(out_a), ref, "attention in front of the projection")
    # the entry point's default is the same pair of launches
    kc, vc, out_d, res_d = fresh()
    assert ops.mha_decode_append(qd, kd, vd, w_d, sin_d, cos_d, kc, vc, out_d, ws, o_weight=wo_d, residual=res_d, **kw) == 2
    torch.cuda.synchronize()
    assert torch.equal(out_d, out_a) and torch.equal(res_d, res_a)
    for call in range(3):
        kc, vc, out_b, res_b = fresh()
        launches = ops.mha_decode_append(qd, kd, vd, w_d, sin_d, cos_d, kc, vc, out_b, ws, o_weight=wo_d, residual=res_b,
                                         one_launch=True, **kw)
        torch.cuda.synchronize()
        assert launches == want_launches
        # The one-launch form may ask for more splits than the dispatcher would pick on its own (it needs idle
        # workgroups): the attention output is then the oracle's within the gate instead of the two-call form's bits,
        # and the residual is, bit for bit, what the GEMV makes of that output.
        assert_parity(from_dev_bf16(out_b), ref, "call %d: attention inside the one-launch form" % call)
        res_chk = to_dev(res0, dev)
        ops.gemv(out_b, wo_d.view(hidden, dim), res_chk, mode=B.GEMV_ADD_BF16)
        torch.cuda.synchronize()
        assert torch.equal(res_b, res_chk), "call %d: residuals differ" % call
        if "num_splits" in extra or launches == 2:
            assert torch.equal(out_b, out_a), "call %d: attention outputs differ" % call
            assert torch.equal(res_b, res_a), "call %d: residuals differ" % call
    n = ctypes.c_uint64()
    assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(n)) == 0


def test_one_launch_projection_that_gives_up_leaves_the_residual_alone(dev):
    """The one-launch form with the poll limit forced to zero: every wait gives up at once, every kernel still ends
    normally, the attention output is poisoned (NaN), the in-place residual stream keeps its bits, and the give-ups are
    counted. With the limit restored the next call on the same workspace matches the pair of launches."""
    n_q, n_kv, d, ctx, hidden = 32, 8, 128, 4096, 2560
    rng = np.random.RandomState(5)
    msl, pos, kv_dim, dim = ctx + 2, ctx, n_kv * d, n_q * d
    case = synth.make_case(901, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
    bits = lambda *shape, scale=1.0: synth.f32_to_bf16_bits((scale * rng.standard_normal(shape)).astype(np.float32))
    q_raw, k_new, v_new = bits(n_q * d), bits(kv_dim), bits(kv_dim)
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    wo, res0 = bits(hidden * dim, scale=1 / np.sqrt(dim)), bits(hidden)
    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    wo_d, w_d, qd, kd, vd = (to_dev(x, dev) for x in (wo, w, q_raw, k_new, v_new))
    ws = torch.full((ops.workspace_bytes(n_q, d, msl) // 4,), float("nan"), dtype=torch.float32, device=dev)
    kw = dict(layer_id=0, pos=pos, kv_dim=kv_dim, kv_mul=n_q // n_kv, head_num=n_q, head_dim=d, max_seq_len=msl,
              kv_layout=B.KV_LAYOUT_HEAD_MAJOR)

    def run(one_launch):
        kc, vc = to_dev(synth.to_head_major(case["k"], n_kv), dev), to_dev(synth.to_head_major(case["v"], n_kv), dev)
        out, res = torch.zeros(dim, dtype=torch.int16, device=dev), to_dev(res0, dev)
        n = ops.mha_decode_append(qd, kd, vd, w_d, sin_d, cos_d, kc, vc, out, ws, o_weight=wo_d, residual=res, one_launch=one_launch, **kw)
        torch.cuda.synchronize()
        return n, out, res

    def timeouts():
        n = ctypes.c_uint64()
        assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(n)) == 0
        return n.value

    _, out_pair, res_pair = run(False)
    before = timeouts()
    prev = B.lib().llmi_hip_set_poll_limit(0)
    try:
        n, out, res = run(True)
    finally:
        assert B.lib().llmi_hip_set_poll_limit(prev) == 0
    assert n == 1
    assert np.all(np.isnan(from_dev_bf16(out)))
    assert torch.equal(res, to_dev(res0, dev)), "a give-up must not touch the residual stream"
    assert timeouts() > before
    after = timeouts()
    ws.fill_(float("nan"))  # (records of the abandoned launch may have arrived late)
    n, out, res = run(True)
    assert n == 1 and torch.equal(res, res_pair) and timeouts() == after
    assert_parity(from_dev_bf16(out), from_dev_bf16(out_pair), "one launch after a give-up")


def test_mha_op_forward_through_registry_hook(oracle, dev):
    """op::MultiHeadAttention::forward (C++ op layer -> registry -> HIP arm) on borrowed device tensors."""
    H = HostLib()
    case = synth.make_case(61, n_q=32, n_kv=8, ctx=1111, max_seq_len=1200, layers=2, layer_id=1)
    ref = oracle.mha_cpu(case["q"], case["k"], case["v"], 1, 1110, 1024, 4, 32, 128, 1200)
    q, k, v = to_dev(case["q"], dev), to_dev(case["k"], dev), to_dev(case["v"], dev)
    out = torch.zeros(32 * 128, dtype=torch.int16, device=dev)
    ws = torch.empty(32 * 4 * 1200, dtype=torch.float32, device=dev)  # the reference's [head_num, 4*max_seq_len]
    rc = H.L.llmi_host_mha_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), ws.data_ptr(), ws.numel(),
                                   out.data_ptr(), 2, 1, 1110, 1024, 4, 32, 128, 1200, 3)
    assert rc == 0, H.L.llmi_host_last_error().decode()
    assert_parity(from_dev_bf16(out), ref, "op layer forward")
    # a workspace smaller than the op's check() accepts is an InvalidArgument status (7), not a launch
    rc = H.L.llmi_host_mha_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), ws.data_ptr(), 32 * 100,
                                   out.data_ptr(), 2, 1, 1110, 1024, 4, 32, 128, 1200, 3)
    assert rc == 7
