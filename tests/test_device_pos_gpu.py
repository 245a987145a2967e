"""GPU tests of the position read from device memory (`llmi_mha_args.pos_device`): one launch, planned for
the largest position, serves every shorter context, eagerly and as a captured graph that is replayed
token after token; against the CPU oracle evaluated at each position."""
import ctypes

import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import assert_parity, assert_tap_parity, from_dev_bf16, to_dev

pytestmark = pytest.mark.gpu


def _oracle_at(oracle, case, pos):
    return oracle.mha_cpu(case["q"], case["k"], case["v"], case["layer_id"], pos, case["kv_dim"], case["kv_mul"],
                          case["head_num"], case["head_dim"], case["max_seq_len"])


@pytest.mark.parametrize("layout", [B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])
@pytest.mark.parametrize("n_q,max_pos,path,splits", [
    (32, 2999, B.PATH_AUTO, 0), (32, 700, B.PATH_SPLIT_FUSED, 11), (64, 1500, B.PATH_AUTO, 0),
    (32, 199, B.PATH_AUTO, 0), (16, 900, B.PATH_SINGLE_PASS, 0),
])
def test_eager_calls_follow_the_device_position(oracle, dev, layout, n_q, max_pos, path, splits):
    """The launch is planned for max_pos; the position tensor then walks over tile, wave and split
    boundaries. Rows beyond the device position hold real data here (a longer history), so reading
    too far shows up as a wrong result, reading beyond max_pos as NaN."""
    n_kv = 8
    case = synth.make_case(900 + max_pos, n_q=n_q, n_kv=n_kv, ctx=max_pos + 1, max_seq_len=max_pos + 5, layers=2,
                           layer_id=1)
    hm = layout == B.KV_LAYOUT_HEAD_MAJOR
    q_d = to_dev(case["q"], dev)
    k_d = to_dev(synth.to_head_major(case["k"], n_kv) if hm else case["k"], dev)
    v_d = to_dev(synth.to_head_major(case["v"], n_kv) if hm else case["v"], dev)
    out = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
    out32 = torch.zeros(n_q * 128, dtype=torch.float32, device=dev)
    ws = torch.full((ops.workspace_bytes(n_q, 128, case["max_seq_len"]) // 4,), float("nan"), dtype=torch.float32,
                    device=dev)
    pos_t = torch.zeros(1, dtype=torch.int32, device=dev)
    scal = dict(layer_id=1, pos=max_pos, kv_dim=case["kv_dim"], kv_mul=case["kv_mul"], head_num=n_q, head_dim=128,
                max_seq_len=case["max_seq_len"], kv_layout=layout, force_path=path, num_splits=splits)
    positions = sorted({0, 1, 15, 16, 17, 63, 64, 65, 239, 240, 241, max_pos // 2, max_pos - 16, max_pos - 1, max_pos}
                       & set(range(max_pos + 1)))
    for p in positions:
        pos_t.fill_(p)
        out.zero_()
        ops.mha_decode(q_d, k_d, v_d, out, ws, output_f32=out32, pos_device=pos_t, **scal)
        torch.cuda.synchronize()
        ref = _oracle_at(oracle, case, p)
        assert_parity(from_dev_bf16(out), ref, "device pos %d of %d" % (p, max_pos))
        assert_tap_parity(out32.cpu().numpy(), ref, "device pos %d of %d" % (p, max_pos))
    # a position beyond the planned one is clamped to it
    pos_t.fill_(max_pos + 3)
    ops.mha_decode(q_d, k_d, v_d, out, ws, pos_device=pos_t, **scal)
    torch.cuda.synchronize()
    assert_parity(from_dev_bf16(out), _oracle_at(oracle, case, max_pos), "clamped position")
    pos_t.fill_(-5)
    ops.mha_decode(q_d, k_d, v_d, out, ws, pos_device=pos_t, **scal)
    torch.cuda.synchronize()
    assert_parity(from_dev_bf16(out), _oracle_at(oracle, case, 0), "negative position clamps to 0")


def test_one_graph_serves_successive_tokens(oracle, dev):
    """A captured launch is replayed while the position tensor and the query change between replays;
    every replay is checked (the workspace keeps the records of the previous replay: same epoch)."""
    n_q, n_kv, max_pos = 32, 8, 2100
    case = synth.make_case(77, n_q=n_q, n_kv=n_kv, ctx=max_pos + 1, max_seq_len=max_pos + 1)
    q_d = to_dev(case["q"], dev)
    k_d = to_dev(synth.to_head_major(case["k"], n_kv), dev)
    v_d = to_dev(synth.to_head_major(case["v"], n_kv), dev)
    out = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
    ws = torch.zeros(ops.workspace_bytes(n_q, 128, max_pos + 1) // 4, dtype=torch.float32, device=dev)
    pos_t = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()
    args = ops.make_mha_args(q_d, k_d, v_d, out, ws, layer_id=0, pos=max_pos, kv_dim=case["kv_dim"],
                             kv_mul=case["kv_mul"], head_num=n_q, head_dim=128, max_seq_len=max_pos + 1,
                             kv_layout=B.KV_LAYOUT_HEAD_MAJOR, pos_device=pos_t, stream=stream.cuda_stream)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        B.check(ops.mha_decode_raw(args), "eager")
        stream.synchronize()
        with torch.cuda.graph(g, stream=stream):
            B.check(ops.mha_decode_raw(args), "capture")
    rng = np.random.RandomState(5)
    for p in [2047, 2048, 2049, 300, 31, 2100, 1024, 1025]:
        q = synth.f32_to_bf16_bits(rng.standard_normal(n_q * 128).astype(np.float32))
        with torch.cuda.stream(stream):
            q_d.copy_(to_dev(q, dev))
            pos_t.fill_(p)
            g.replay()
        stream.synchronize()
        c = dict(case, q=q)
        assert_parity(from_dev_bf16(out), _oracle_at(oracle, c, p), "replay at pos %d" % p)


@pytest.mark.parametrize("layout,n_q,start", [(B.KV_LAYOUT_POS_MAJOR, 32, 250), (B.KV_LAYOUT_HEAD_MAJOR, 32, 250),
                                               (B.KV_LAYOUT_HEAD_MAJOR, 16, 65533)])
def test_append_graph_decodes_token_after_token(oracle, dev, layout, n_q, start):
    """llmi_hip_mha_decode_append captured once with a device position: every replay normalises and
    rotates with the sin/cos row of its own position, appends K/V at its own slot and attends over the
    rows appended so far. The oracle replays the same chain on the host. (The long case walks over 65536 cached
    positions, where the splits' runs are 512 KiB long: the kernel, which only learns the length on the device,
    staggers its walk from there on and not before.)"""
    n_kv, d, tokens = 8, 128, 6
    msl = start + tokens + 2
    kv_dim = n_kv * d
    case = synth.make_case(31, n_q=n_q, n_kv=n_kv, ctx=start, max_seq_len=msl)
    k_host, v_host = case["k"].copy(), case["v"].copy()
    hm = layout == B.KV_LAYOUT_HEAD_MAJOR
    k_d = to_dev(synth.to_head_major(k_host, n_kv) if hm else k_host, dev)
    v_d = to_dev(synth.to_head_major(v_host, n_kv) if hm else v_host, dev)
    rng = np.random.RandomState(8)
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * d)).astype(np.float32))
    w_d = to_dev(w, dev)
    sin_o, cos_o = oracle.sincos_table(d, msl)
    sin_d, cos_d = ops.sincos_table(d, msl, dev)
    q_d = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    kn_d = torch.zeros(kv_dim, dtype=torch.int16, device=dev)
    vn_d = torch.zeros(kv_dim, dtype=torch.int16, device=dev)
    out = torch.zeros(n_q * d, dtype=torch.int16, device=dev)
    ws = torch.zeros(ops.workspace_bytes(n_q, d, msl) // 4, dtype=torch.float32, device=dev)
    pos_t = torch.full((1,), start, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()

    a = B.MhaAppendArgs()
    a.mha = ops.make_mha_args(q_d, k_d, v_d, out, ws, layer_id=0, pos=msl - 1, kv_dim=kv_dim, kv_mul=n_q // n_kv,
                              head_num=n_q, head_dim=d, max_seq_len=msl, kv_layout=layout, pos_device=pos_t,
                              stream=stream.cuda_stream)
    a.key_new, a.value_new, a.norm_weight = kn_d.data_ptr(), vn_d.data_ptr(), w_d.data_ptr()
    a.sin_cache, a.cos_cache, a.eps = sin_d.data_ptr(), cos_d.data_ptr(), 1e-6
    call = B.lib().llmi_hip_mha_decode_append

    def feed(p):
        q = synth.f32_to_bf16_bits(rng.standard_normal((n_q, d)).astype(np.float32))
        kn = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
        vn = synth.f32_to_bf16_bits(rng.standard_normal((n_kv, d)).astype(np.float32))
        q_d.copy_(to_dev(q.reshape(-1), dev))
        kn_d.copy_(to_dev(kn.reshape(-1), dev))
        vn_d.copy_(to_dev(vn.reshape(-1), dev))
        pos_t.fill_(p)
        k_host[0, p] = oracle.qk_norm_rope(kn, w[d:], sin_o[p], cos_o[p]).reshape(-1)
        v_host[0, p] = vn.reshape(-1)
        q_n = oracle.qk_norm_rope(q, w[:d], sin_o[p], cos_o[p])
        return oracle.mha_cpu(q_n.reshape(-1), k_host, v_host, 0, p, kv_dim, n_q // n_kv, n_q, d, msl)

    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        ref = feed(start)
        B.check(call(ctypes.byref(a)), "eager append")
        stream.synchronize()
        assert_parity(from_dev_bf16(out), ref, "eager append at %d" % start)
        with torch.cuda.graph(g, stream=stream):
            B.check(call(ctypes.byref(a)), "capture append")
    for p in range(start + 1, start + tokens):
        with torch.cuda.stream(stream):
            ref = feed(p)
            g.replay()
        stream.synchronize()
        assert_parity(from_dev_bf16(out), ref, "append replay at %d" % p)
    kc = k_d.cpu().numpy().view(np.uint16)
    if hm:
        kc = np.ascontiguousarray(kc.transpose(0, 2, 1, 3)).reshape(1, msl, kv_dim)
    last = start + tokens - 1
    got = synth.bf16_bits_to_f32(kc[0, start:last + 1]).astype(np.float64)
    want = synth.bf16_bits_to_f32(k_host[0, start:last + 1]).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.abs(want) / 128 + 1e-6)
    assert np.all(kc[0, last + 1:] == 0x7FC0)  # nothing beyond the last appended row was written


def test_device_position_at_lengths_with_and_without_the_staggered_walk(oracle, dev):
    """Head-major, planned for 70001 positions (the longest run exceeds 512 KiB, so the launch uses the kernels that can
    stagger their walk); the device position then visits lengths where the rule applies (65536 exactly, a few tiles
    above) and where it does not (below, in between): every result is the oracle's."""
    n_q, n_kv, max_pos = 16, 8, 70000
    case = synth.make_case(77, n_q=n_q, n_kv=n_kv, ctx=max_pos + 1, max_seq_len=max_pos + 1)
    q_d = to_dev(case["q"], dev)
    k_d = to_dev(synth.to_head_major(case["k"], n_kv), dev)
    v_d = to_dev(synth.to_head_major(case["v"], n_kv), dev)
    out = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
    out32 = torch.zeros(n_q * 128, dtype=torch.float32, device=dev)
    ws = torch.full((ops.workspace_bytes(n_q, 128, case["max_seq_len"]) // 4,), float("nan"), dtype=torch.float32, device=dev)
    pos_t = torch.zeros(1, dtype=torch.int32, device=dev)
    scal = dict(layer_id=0, pos=max_pos, kv_dim=case["kv_dim"], kv_mul=case["kv_mul"], head_num=n_q, head_dim=128,
                max_seq_len=case["max_seq_len"], kv_layout=B.KV_LAYOUT_HEAD_MAJOR)
    for side in (0, ops.workspace_side(ws) or 0x55555555):
        for p in (65535, 65535 + 37, 65535 + 16 * 8 * 32, 50000, 3000, max_pos):  # (+4096: eight tiles per run above the multiple)
            pos_t.fill_(p)
            out.zero_()
            ops.mha_decode(q_d, k_d, v_d, out, ws, output_f32=out32, pos_device=pos_t, workspace_side=side, **scal)
            torch.cuda.synchronize()
            ref = _oracle_at(oracle, case, p)
            assert_parity(from_dev_bf16(out), ref, "device pos %d, side %x" % (p, side))
            assert_tap_parity(out32.cpu().numpy(), ref, "device pos %d, side %x" % (p, side))


def test_plan_rejects_device_position_with_separate_combine(dev):
    pos_t = torch.zeros(1, dtype=torch.int32, device=dev)
    t = torch.zeros(32 * 128, dtype=torch.int16, device=dev)
    kv = torch.zeros(1, 512, 1024, dtype=torch.int16, device=dev)
    ws = torch.zeros(1 << 20, dtype=torch.float32, device=dev)
    a = ops.make_mha_args(t, kv, kv, t, ws, layer_id=0, pos=511, kv_dim=1024, kv_mul=4, head_num=32, head_dim=128,
                          max_seq_len=512, force_path=B.PATH_SPLIT, num_splits=4, pos_device=pos_t)
    assert ops.mha_decode_raw(a) == B.STATUS["INVALID_ARG"]
