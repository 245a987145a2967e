"""The engine's weight file (8 x int32 header + flat bf16 payload, tools/qwen3/qwen3_dense_unified_converter.py:43-57)
read by model::WeightFile: header, derived sizes, payload length check, tensor offsets (CPU), and the attention
block's weights loaded into the captured stack (GPU)."""
import ctypes
import os

import numpy as np
import pytest

from llminfer_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIXTURE = os.path.join(ROOT, "tests", "golden", "engine_loader_fixture_7int_header.bin")


def host_lib():
    L = ctypes.CDLL(os.path.join(ROOT, "llminfer_amd", "libllmi_host.so"))
    L.llmi_host_last_error.restype = ctypes.c_char_p
    L.llmi_host_weight_file_info.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_int64),
                                             ctypes.c_void_p, ctypes.c_int64]
    return L


def info(L, path, header_ints=8, payload_bytes=0):
    out = (ctypes.c_int64 * 12)()
    buf = np.zeros(max(payload_bytes, 1), dtype=np.uint8)
    rc = L.llmi_host_weight_file_info(path.encode(), header_ints, out, buf.ctypes.data_as(ctypes.c_void_p), payload_bytes)
    return rc, list(out), buf[:payload_bytes]


def sections(cfg):
    """(name, per-layer shape, layers) in file order: qwen3_fused.cpp:246-314."""
    dim, hid, L, hn, kvh, vocab, _, imm = cfg
    hd = dim // hn
    kv = hd * kvh
    return [("embedding", (abs(vocab), hid), 1), ("pre_rmsnorm", (hid,), L), ("qkv", (dim + 2 * kv, hid), L),
            ("qk_norm", (2 * hd,), L), ("o_proj", (hid, dim), L), ("ffn_rmsnorm", (hid,), L),
            ("gate_up", (2 * imm, hid), L), ("down", (hid, imm), L), ("final_rmsnorm", (hid,), 1)]


def write_weight_file(path, cfg, seed=0, scale=None):
    """Writes a file in the engine's format; returns {name: uint16 array [layers, ...]}."""
    rng = np.random.RandomState(seed)
    tensors = {}
    with open(path, "wb") as f:
        f.write(np.asarray(cfg, dtype=np.int32).tobytes())
        for name, shape, layers in sections(cfg):
            x = rng.standard_normal((layers,) + shape).astype(np.float32)
            if name.endswith("norm"):
                x = 1 + 0.02 * x
            elif len(shape) == 2:
                x = x / np.sqrt(shape[1])
            bits = synth.f32_to_bf16_bits(x)
            tensors[name] = bits
            f.write(bits.tobytes())
    return tensors


def test_header_and_derived_sizes(tmp_path):
    L = host_lib()
    cfg = (256, 64, 2, 2, 1, 8, 32, 96)  # dim, hidden, layers, heads, kv heads, vocab, max_seq_len, immediate
    p = str(tmp_path / "w.bin")
    t = write_weight_file(p, cfg)
    rc, out, payload = info(L, p, payload_bytes=8 * 64 * 2)
    assert rc == 0, L.llmi_host_last_error().decode()
    assert tuple(out[:8]) == cfg
    assert out[8] == 128 and out[9] == 128 and out[10] == 8
    assert out[11] == sum(int(np.prod(s)) * n for _, s, n in sections(cfg))
    assert np.array_equal(payload.view(np.uint16), t["embedding"].reshape(-1))  # the payload starts right after the header


def test_negative_vocab_size_means_untied_but_same_size(tmp_path):
    L = host_lib()
    cfg = (256, 64, 1, 2, 1, -8, 32, 96)  # model.cpp:229-233: the sign is a flag, |vocab_size| sizes the embedding
    p = str(tmp_path / "w.bin")
    write_weight_file(p, cfg)
    rc, out, _ = info(L, p)
    assert rc == 0 and out[5] == -8 and out[10] == 8


@pytest.mark.parametrize("delta", [-2, 2, 4096])
def test_payload_length_must_match_the_header(tmp_path, delta):
    """qwen3_fused.cpp:317-318: consumed bytes == file size."""
    L = host_lib()
    p = str(tmp_path / "w.bin")
    write_weight_file(p, (256, 64, 2, 2, 1, 8, 32, 96))
    data = open(p, "rb").read()
    open(p, "wb").write(data[:delta] if delta < 0 else data + b"\0" * delta)
    rc, _, _ = info(L, p)
    assert rc == 3 and b"bytes" in L.llmi_host_last_error()  # ModelParseError


def test_bad_paths_and_headers(tmp_path):
    L = host_lib()
    assert info(L, str(tmp_path / "missing.bin"))[0] == 2          # PathNotValid (model.cpp:136-139)
    assert info(L, "")[0] == 2                                     # :131-133
    p = str(tmp_path / "short.bin")
    open(p, "wb").write(b"\1\0\0\0" * 5)
    assert info(L, p)[0] == 3                                      # header cut short (:148-150)
    q = str(tmp_path / "odd.bin")
    open(q, "wb").write(np.asarray((250, 64, 1, 3, 1, 8, 32, 96), dtype=np.int32).tobytes())
    assert info(L, q)[0] == 3                                      # dim % head_num != 0 (:221)


@pytest.mark.parametrize("cfg", [
    (256, 64, 2, 2, 1, -2**31, 32, 96),                     # |vocab_size| does not exist
    (2**30, 2**30, 2**30, 2, 1, 2**30, 32, 2**30),          # every product wraps 64 bits
    (2**16, 2**31 - 1, 2**31 - 1, 1, 1, 2**31 - 1, 32, 2**31 - 1),
    (2**31 - 2, 64, 1, 2, 2**31 - 1, 8, 32, 96),            # head_dim * kv_head_num beyond int32
    (256, 64, 2**31 - 1, 2, 1, 8, 32, 96),                  # plausible shapes, absurd layer count
])
def test_overflowing_headers_are_parse_errors(tmp_path, cfg):
    """The header is untrusted: sizes that wrap 32- or 64-bit arithmetic must not pass the length check
    (they could make the summed offsets wrap round to the real file size), whatever payload follows."""
    L = host_lib()
    p = str(tmp_path / "evil.bin")
    with open(p, "wb") as f:
        f.write(np.asarray(cfg, dtype=np.int64).astype(np.int32).tobytes())
        f.write(b"\0" * 4096)
    rc, _, _ = info(L, p)
    assert rc == 3, L.llmi_host_last_error().decode()


def test_engine_fixture_with_the_older_header():
    """The engine's own loader fixture (7 x int32 header, then float(i) for i < dim * hidden_dim): the values its
    test expects (test/test_op/test_load.cpp:19-26,52-56)."""
    L = host_lib()
    rc, out, payload = info(L, FIXTURE, header_ints=7, payload_bytes=2048 * 4)
    assert rc == 0, L.llmi_host_last_error().decode()
    dim, hidden, layers, heads, kv_heads, vocab, msl = out[:7]
    assert (dim, hidden, layers, heads, kv_heads, vocab, msl) == (16, 128, 256, 512, 512, 4, 1024)
    assert out[7] == 0 and out[10] == 4 and os.path.getsize(FIXTURE) == 7 * 4 + 2048 * 4
    assert np.array_equal(payload.view(np.float32), np.arange(2048, dtype=np.float32))


@pytest.mark.gpu
def test_stack_runs_the_attention_block_from_a_weight_file(tmp_path, oracle, dev):
    """Two layers of a 16 Q / 8 KV head model written to disk, loaded into the stack, run as mode 3; the oracle
    chain uses the arrays that were written."""
    from llminfer_amd import _binding as B
    from helpers import assert_parity
    L = host_lib()
    L.llmi_host_stack_create.restype = ctypes.c_void_p
    L.llmi_host_stack_create.argtypes = [ctypes.c_int32] * 5
    L.llmi_host_stack_destroy.argtypes = [ctypes.c_void_p]
    L.llmi_host_stack_ptr.restype = ctypes.c_void_p
    L.llmi_host_stack_ptr.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    L.llmi_host_stack_build_sincos.argtypes = [ctypes.c_void_p]
    L.llmi_host_stack_run.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    L.llmi_host_stack_load_weights.argtypes = [ctypes.c_void_p, ctypes.c_char_p]

    def up(ptr, arr):
        arr = np.ascontiguousarray(arr)
        assert B.lib().llmi_hip_memcpy(ptr, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes, 1, None, 1) == 0

    def down(ptr, shape):
        out = np.empty(shape, dtype=np.uint16)
        assert B.lib().llmi_hip_memcpy(out.ctypes.data_as(ctypes.c_void_p), ptr, out.nbytes, 2, None, 1) == 0
        return out

    n_q, n_kv, d, hidden, layers, ctx = 16, 8, 128, 1024, 3, 260
    dim, kv_dim, msl, pos = n_q * d, n_kv * d, ctx + 1, ctx
    path = str(tmp_path / "model.bin")
    t = write_weight_file(path, (dim, hidden, layers, n_q, n_kv, 4, 4096, 256), seed=3)
    stack = L.llmi_host_stack_create(2, msl, n_q, n_kv, B.KV_LAYOUT_HEAD_MAJOR)  # the stack uses the first 2 layers
    assert stack
    try:
        assert L.llmi_host_stack_load_weights(stack, path.encode()) == 0, L.llmi_host_last_error().decode()
        assert L.llmi_host_stack_load_weights(stack, (path + ".nope").encode()) == 2
        assert L.llmi_host_stack_build_sincos(stack) == 0
        rng = np.random.RandomState(2)
        sin_o, cos_o = oracle.sincos_table(d, msl)
        res0 = synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32))
        res_ref = synth.bf16_bits_to_f32(res0).copy()
        k_all = np.zeros((2, msl, kv_dim), dtype=np.uint16)
        v_all = np.zeros((2, msl, kv_dim), dtype=np.uint16)
        refs = []
        for l in range(2):
            c = synth.make_case(60 + l, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=msl)
            k_all[l], v_all[l] = c["k"][0], c["v"][0]
            x = synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32))
            up(L.llmi_host_stack_ptr(stack, 12, l), x)
            w = t["qk_norm"][l]
            qkv = synth.f32_to_bf16_bits(oracle.gemv_bf16(x, t["qkv"][l]))
            k_all[l, pos] = oracle.qk_norm_rope(qkv[dim:dim + kv_dim].reshape(n_kv, d), w[d:], sin_o[pos], cos_o[pos]).reshape(-1)
            v_all[l, pos] = qkv[dim + kv_dim:]
            qn = oracle.qk_norm_rope(qkv[:dim].reshape(n_q, d), w[:d], sin_o[pos], cos_o[pos]).reshape(-1)
            attn = oracle.mha_cpu(qn, k_all[l:l + 1], v_all[l:l + 1], 0, pos, kv_dim, n_q // n_kv, n_q, d, msl)
            refs.append(attn)
            res_ref = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(
                res_ref + oracle.gemv_bf16(synth.f32_to_bf16_bits(attn), t["o_proj"][l])))
        k_up, v_up = k_all.copy(), v_all.copy()
        k_up[:, pos], v_up[:, pos] = 0x7FC0, 0x7FC0
        up(L.llmi_host_stack_ptr(stack, 0, 0), synth.to_head_major(k_up, n_kv))
        up(L.llmi_host_stack_ptr(stack, 1, 0), synth.to_head_major(v_up, n_kv))
        up(L.llmi_host_stack_ptr(stack, 13, 0), res0)
        assert L.llmi_host_stack_run(stack, pos, 3) == 0, L.llmi_host_last_error().decode()
        for l in range(2):
            got = down(L.llmi_host_stack_ptr(stack, 6, l), (n_q * d,))
            assert_parity(synth.bf16_bits_to_f32(got), refs[l], "layer %d from file" % l)
        res = synth.bf16_bits_to_f32(down(L.llmi_host_stack_ptr(stack, 13, 0), (hidden,)))
        assert np.all(np.abs(res - res_ref) <= np.abs(res_ref) / 64 + 2e-2)
        # the weights on the device are the file's bytes
        assert np.array_equal(down(L.llmi_host_stack_ptr(stack, 10, 1), t["qkv"][1].shape), t["qkv"][1])
        assert np.array_equal(down(L.llmi_host_stack_ptr(stack, 11, 1), t["o_proj"][1].shape), t["o_proj"][1])
    finally:
        L.llmi_host_stack_destroy(stack)
