"""Pins the CPU oracle (oracle/llmi_oracle.c) without the reference: golden vectors made by an
independent float64 evaluation, library routines (torch SDPA, torch bf16 conversion, scipy softmax),
closed forms, invariants and long-double brute force. Each check is chosen so that a plausible slip
(dropped scale, wrong KV-head index, transposed operand, off-by-one in pos, wrong rotation sign) fails it."""
import os

import numpy as np
import pytest
import torch

import make_golden
from llminfer_amd import synth


# ---------------------------------------------------------------- bf16 helpers
def test_bf16_round_trip_all_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.bf16_to_f32(bits)
    back = oracle.f32_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], bits[~nan])


def test_bf16_rne_ties_and_known_values(oracle):
    def conv(u32):
        return int(oracle.f32_to_bf16(np.array([u32], dtype=np.uint32).view(np.float32))[0])
    assert conv(0x3F808000) == 0x3F80  # tie -> even (down)
    assert conv(0x3F818000) == 0x3F82  # tie -> even (up)
    assert conv(0x3F808001) == 0x3F81  # just above the tie
    assert conv(0x3F807FFF) == 0x3F80
    assert conv(0x3F800000) == 0x3F80  # 1.0
    assert conv(0xC0490FDB) == 0xC049  # -pi


def test_bf16_matches_torch_and_synth(oracle):
    x = np.random.RandomState(0).standard_normal(200000).astype(np.float32) * 37.0
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(x), want)
    assert np.array_equal(synth.f32_to_bf16_bits(x), want)
    assert np.array_equal(synth.bf16_bits_to_f32(want), oracle.bf16_to_f32(want))


# ---------------------------------------------------------------- softmax (C3)
@pytest.mark.parametrize("n", [1, 2, 7, 64])
def test_softmax_brute_force_long_double(oracle, n):
    x = (np.random.RandomState(n).standard_normal(n) * 4).astype(np.float32)
    xl = x.astype(np.longdouble)
    e = np.exp(xl - xl.max())
    want = (e / e.sum()).astype(np.float64)
    got = oracle.softmax(x).astype(np.float64)
    assert np.allclose(got, want, rtol=5e-6, atol=1e-9)


def test_softmax_invariants(oracle):
    x = (np.random.RandomState(3).standard_normal(257) * 3).astype(np.float32)
    p = oracle.softmax(x)
    assert abs(float(p.sum(dtype=np.float64)) - 1.0) < 1e-5
    assert np.allclose(oracle.softmax(x + np.float32(5.0)), p, rtol=2e-5, atol=1e-9)  # shift invariance
    assert oracle.softmax(np.array([3.25], dtype=np.float32))[0] == 1.0
    assert np.allclose(oracle.softmax(np.full(10, -2.0, dtype=np.float32)), 0.1, rtol=1e-6)
    assert np.argmax(p) == np.argmax(x)


# ---------------------------------------------------------------- scores (C2)
def test_dot_scaled_closed_forms(oracle):
    k = np.random.RandomState(4).standard_normal(128).astype(np.float32)
    scale = np.float32(2.0 ** -3.5)  # 1/sqrt(128)
    for i in (0, 5, 127):
        e = np.zeros(128, dtype=np.float32)
        e[i] = 1.0
        assert oracle.dot_scaled(e, k, float(scale)) == pytest.approx(float(np.float32(k[i]) * scale), rel=1e-7)
    q = np.random.RandomState(5).standard_normal(128).astype(np.float32)
    want = float(np.dot(q.astype(np.float64), k.astype(np.float64))) * float(scale)
    assert oracle.dot_scaled(q, k, float(scale)) == pytest.approx(want, rel=1e-5, abs=1e-6)
    assert oracle.dot_scaled(q, k, 1.0) == pytest.approx(oracle.dot_scaled(k, q, 1.0), rel=1e-6)


# ---------------------------------------------------------------- weighted sum (C4)
def test_scale_sum_closed_forms(oracle):
    rng = np.random.RandomState(6)
    pos, d, kv_dim = 40, 128, 1024
    p = oracle.softmax(rng.standard_normal(pos + 1).astype(np.float32))
    v_row = rng.standard_normal(d).astype(np.float32)
    value = np.zeros((pos + 1, kv_dim), dtype=np.float32)
    value[:, :d] = v_row  # all rows equal -> out = v * sum(p)
    out = oracle.scale_sum(p, value.reshape(-1), pos, d, kv_dim)
    assert np.allclose(out, v_row * p.sum(dtype=np.float64), rtol=1e-5, atol=1e-6)
    # one-hot weights pick one row, and the stride between rows is kv_dim, not head_dim
    value = rng.standard_normal((pos + 1, kv_dim)).astype(np.float32)
    hot = np.zeros(pos + 1, dtype=np.float32)
    hot[17] = 1.0
    assert np.array_equal(oracle.scale_sum(hot, value.reshape(-1), pos, d, kv_dim), value[17, :d])
    # accumulates into out (the caller zeroes it first)
    base = np.ones(d, dtype=np.float32)
    assert np.array_equal(oracle.scale_sum(hot, value.reshape(-1), pos, d, kv_dim, out=base.copy()), value[17, :d] + 1)


# ---------------------------------------------------------------- the op (C1)
@pytest.mark.parametrize("name", sorted(make_golden.RECIPES))
def test_mha_cpu_golden(oracle, name):
    """Golden vectors: float64 einsum/scipy evaluation, made without the oracle."""
    c = make_golden.load(name)
    k, v = c["k"], c["v"]
    if k.dtype == np.uint16:  # NaN-pattern padding outside the live rows stays in place: it must never be read
        pass
    got = oracle.mha_cpu(c["q"], k, v, c["layer_id"], c["pos"], c["n_kv"] * c["head_dim"], c["n_q"] // c["n_kv"],
                         c["n_q"], c["head_dim"], c["max_seq_len"])
    assert np.all(np.isfinite(got))
    assert np.allclose(got, c["expected"], rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("n_q,n_kv,pos,layers,layer_id,msl", [
    (16, 8, 256, 1, 0, 512),   # the CPU-plumbing configuration
    (4, 2, 12, 10, 3, 256),    # shapes of the reference's own op test (test_op_mha.cpp:9-18), head_dim 128
    (16, 4, 12, 10, 7, 256),   # test_op_mha.cpp:68-78
    (8, 8, 40, 2, 1, 64),      # kv_mul 1
    (8, 1, 33, 1, 0, 34),      # one KV head for all (MQA), pos = max_seq_len-1
])
def test_mha_cpu_matches_torch_sdpa_fp64(oracle, n_q, n_kv, pos, layers, layer_id, msl):
    """The textbook routine: torch.nn.functional.scaled_dot_product_attention in float64."""
    rng = np.random.RandomState(n_q * 1000 + pos)
    d = 128
    q = rng.standard_normal(n_q * d).astype(np.float32)
    k = rng.standard_normal((layers, msl, n_kv * d)).astype(np.float32)  # every layer and row filled:
    v = rng.standard_normal((layers, msl, n_kv * d)).astype(np.float32)  # a wrong layer/row gives wrong numbers
    got = oracle.mha_cpu(q, k, v, layer_id, pos, n_kv * d, n_q // n_kv, n_q, d, msl)
    L = pos + 1
    qt = torch.from_numpy(q).double().reshape(1, n_q, 1, d)
    kt = torch.from_numpy(k[layer_id, :L]).double().reshape(L, n_kv, d).permute(1, 0, 2)
    vt = torch.from_numpy(v[layer_id, :L]).double().reshape(L, n_kv, d).permute(1, 0, 2)
    kt = kt.repeat_interleave(n_q // n_kv, dim=0).unsqueeze(0)
    vt = vt.repeat_interleave(n_q // n_kv, dim=0).unsqueeze(0)
    want = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt).reshape(-1).numpy()
    assert np.allclose(got, want, rtol=2e-5, atol=2e-6)


def test_mha_cpu_score_buffer_holds_softmax_weights(oracle):
    c = make_golden.load("cfg1_fp32_seed1")
    out, score = oracle.mha_cpu(c["q"], c["k"], c["v"], 0, c["pos"], 1024, 2, 16, 128, 512, return_score=True)
    L = c["pos"] + 1
    assert np.allclose(score[:, :L].sum(axis=1, dtype=np.float64), 1.0, atol=1e-5)
    assert np.all(score[:, L:] == 0)  # nothing past pos is touched
    # scale check: score ratios follow exp((s_a - s_b)/sqrt(128)); dropping the scale would change them
    q0 = c["q"][:128].astype(np.float64)
    s = c["k"][0, :L, :128].astype(np.float64) @ q0 / np.sqrt(128.0)
    assert np.allclose(np.log(score[0, 1] / score[0, 0]), s[1] - s[0], atol=1e-4)


def test_mha_cpu_gqa_addressing(oracle):
    """K/V filled with a function of (layer, t, kv_head): heads of one group see the same cache rows."""
    n_q, n_kv, d, msl, layers, pos = 8, 2, 128, 20, 3, 9
    k = np.zeros((layers, msl, n_kv * d), dtype=np.float32)
    v = np.zeros((layers, msl, n_kv * d), dtype=np.float32)
    for l in range(layers):
        for t in range(msl):
            for g in range(n_kv):
                k[l, t, g * d:(g + 1) * d] = 0.01 * (l + 1) * (t + 1) * (1 if g == 0 else -1)
                v[l, t, g * d:(g + 1) * d] = 100 * l + 10 * g + t
    q = np.tile(np.ones(d, dtype=np.float32), n_q)  # identical queries
    out = oracle.mha_cpu(q, k, v, 1, pos, n_kv * d, n_q // n_kv, n_q, d, msl).reshape(n_q, d)
    assert np.allclose(out[0], out[3]) and np.allclose(out[4], out[7])  # same group -> same output
    assert not np.allclose(out[0], out[4])                                # other group differs
    # group 0 has scores growing with t -> mean position > pos/2; group 1 the opposite; layer 1 -> offset 100
    assert 100 + pos / 2 < out[0, 0] < 100 + pos
    assert 110 < out[4, 0] < 110 + pos / 2


def test_mha_cpu_bf16_variant_is_bit_identical_to_widened_fp32(oracle):
    c = synth.make_case(77, n_q=32, n_kv=8, ctx=129, max_seq_len=140, layers=2, layer_id=1, fill_layers="all")
    a = oracle.mha_cpu(c["q"], c["k"], c["v"], 1, c["pos"], 1024, 4, 32, 128, 140)
    kf = synth.bf16_bits_to_f32(c["k"])
    vf = synth.bf16_bits_to_f32(c["v"])
    kf[~np.isfinite(kf)] = 0
    vf[~np.isfinite(vf)] = 0
    b = oracle.mha_cpu(synth.bf16_bits_to_f32(c["q"]), kf, vf, 1, c["pos"], 1024, 4, 32, 128, 140)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("bad", [dict(pos=-1), dict(pos=16), dict(layer_id=-1)])
def test_mha_cpu_rejects_what_the_reference_checks(oracle, bad):
    c = synth.make_case(1, n_q=8, n_kv=2, ctx=16)
    args = dict(layer_id=0, pos=15)
    args.update(bad)
    with pytest.raises(ValueError):
        oracle.mha_cpu(c["q"], c["k"], c["v"], args["layer_id"], args["pos"], 256, 4, 8, 128, 16)


# ---------------------------------------------------------------- split + combine (G3/G4)
@pytest.mark.parametrize("L", [1, 31, 32, 33, 127, 128, 129, 257])
def test_split_combine_equals_single_pass(oracle, L):
    """For any partition of [0, L) the log-sum-exp merge of the partials equals the one-pass result."""
    rng = np.random.RandomState(L)
    d, kv_dim = 128, 256
    q = rng.standard_normal(d).astype(np.float32)
    k = rng.standard_normal((L, kv_dim)).astype(np.float32)
    v = rng.standard_normal((L, kv_dim)).astype(np.float32)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(d)))
    o1, m1, l1 = oracle.split_partial(q, k.reshape(-1), v.reshape(-1), 0, L, d, kv_dim, scale)
    one = oracle.combine(o1[None, :], [m1], [l1])
    assert np.allclose(one, o1 / l1, rtol=1e-6)  # S = 1: the merge is the normalisation
    # fp64 definition
    s = k[:, :d].astype(np.float64) @ q.astype(np.float64) * scale
    p = np.exp(s - s.max())
    want = (p[:, None] * v[:, :d]).sum(0) / p.sum()
    assert np.allclose(one, want, rtol=2e-5, atol=2e-6)
    for cuts in ([L // 2], [1], [L - 1], sorted(set(rng.randint(0, L + 1, size=5).tolist()))):
        edges = [0] + [c for c in cuts if 0 <= c <= L] + [L]
        parts = [oracle.split_partial(q, k.reshape(-1), v.reshape(-1), a, b, d, kv_dim, scale)
                 for a, b in zip(edges[:-1], edges[1:])]  # may contain empty ranges (a == b)
        merged = oracle.combine(np.stack([p_[0] for p_ in parts]), [p_[1] for p_ in parts], [p_[2] for p_ in parts])
        assert np.allclose(merged, one, rtol=1e-5, atol=1e-6)


def test_empty_split_contributes_nothing(oracle):
    d = 128
    q = np.ones(d, dtype=np.float32)
    k = np.ones((4, d), dtype=np.float32)
    o, m, l = oracle.split_partial(q, k.reshape(-1), k.reshape(-1), 2, 2, d, d, 1.0)
    assert m == -np.inf and l == 0.0 and not o.any()


# ---------------------------------------------------------------- sin/cos table, QK-Norm + RoPE
def test_sincos_table_against_long_double(oracle):
    sin, cos = oracle.sincos_table(128, 12346)
    assert np.all(sin[0] == 0) and np.all(cos[0] == 1)  # pos 0: identity rotation
    assert np.allclose(sin.astype(np.float64) ** 2 + cos.astype(np.float64) ** 2, 1.0, atol=1e-6)
    i = np.arange(64, dtype=np.longdouble)
    freq = np.power(np.longdouble(1e6), -2 * i / 128)
    for pos in (1, 4096, 12345):
        theta = np.longdouble(pos) * freq
        # the table multiplies float(pos) by a float frequency: allow that rounding (|theta| * 2^-24)
        tol = 2e-6 + float(pos) * 2.0 ** -23
        assert np.allclose(sin[pos], np.sin(theta).astype(np.float64), atol=tol)
        assert np.allclose(cos[pos], np.cos(theta).astype(np.float64), atol=tol)


def _qk_norm_rope_f64(x_bits, w_bits, sin_row, cos_row, eps):
    """fp64 form of the reference's torch model (test_kernel/test_qwen3_bf16_ops.py:777-794)."""
    x = synth.bf16_bits_to_f32(x_bits).astype(np.float64)
    w = synth.bf16_bits_to_f32(w_bits).astype(np.float64)
    y = x * w[None, :] / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps)
    a, b = y[:, :64], y[:, 64:]
    return np.concatenate([a * cos_row - b * sin_row, a * sin_row + b * cos_row], axis=1)


def test_qk_norm_rope_against_fp64_model(oracle):
    rng = np.random.RandomState(9)
    x = synth.f32_to_bf16_bits(rng.standard_normal((40, 128)).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(128)).astype(np.float32))
    sin, cos = oracle.sincos_table(128, 4097)
    got = synth.bf16_bits_to_f32(oracle.qk_norm_rope(x, w, sin[4096], cos[4096], 1e-6)).astype(np.float64)
    want = _qk_norm_rope_f64(x, w, sin[4096].astype(np.float64), cos[4096].astype(np.float64), 1e-6)
    # one bf16 rounding of the fp32 chain: half an ulp = 2^-9 relative, plus fp32 noise
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-6)
    exact = synth.f32_to_bf16_bits(want.astype(np.float32)) == synth.f32_to_bf16_bits(got.astype(np.float32))
    assert exact.mean() > 0.99


def test_qk_norm_rope_invariants(oracle):
    rng = np.random.RandomState(10)
    xf = rng.standard_normal((8, 128)).astype(np.float32)
    x = synth.f32_to_bf16_bits(xf)
    ones = synth.f32_to_bf16_bits(np.ones(128, dtype=np.float32))
    sin, cos = oracle.sincos_table(128, 1000)
    # pos 0 -> no rotation: pure RMSNorm, output RMS = 1 with unit weights
    y0 = synth.bf16_bits_to_f32(oracle.qk_norm_rope(x, ones, sin[0], cos[0], 1e-6))
    assert np.allclose(np.sqrt((y0.astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=4e-3)
    assert np.all(np.sign(y0) == np.sign(synth.bf16_bits_to_f32(x)))
    # rotation preserves the norm of every (i, i+64) pair
    y = synth.bf16_bits_to_f32(oracle.qk_norm_rope(x, ones, sin[777], cos[777], 1e-6)).astype(np.float64)
    n0 = y0[:, :64].astype(np.float64) ** 2 + y0[:, 64:].astype(np.float64) ** 2
    n1 = y[:, :64] ** 2 + y[:, 64:] ** 2
    assert np.allclose(n0, n1, rtol=2e-2, atol=1e-4)
    # scaling the input by a power of two changes nothing with eps = 0, and next to nothing with eps << mean
    x4 = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(x) * 4.0)
    assert np.array_equal(oracle.qk_norm_rope(x4, ones, sin[777], cos[777], 0.0),
                          oracle.qk_norm_rope(x, ones, sin[777], cos[777], 0.0))
    same = oracle.qk_norm_rope(x4, ones, sin[777], cos[777], 1e-6) == oracle.qk_norm_rope(x, ones, sin[777],
                                                                                          cos[777], 1e-6)
    assert same.mean() > 0.99
    # sign convention: a pure "a" component rotates towards +b for positive sin
    e = np.zeros((1, 128), dtype=np.float32)
    e[0, 3] = 1.0
    r = synth.bf16_bits_to_f32(oracle.qk_norm_rope(synth.f32_to_bf16_bits(e), ones, sin[1], cos[1], 0.0))
    s3, c3 = float(sin[1, 3]), float(cos[1, 3])
    amp = np.sqrt(128.0)  # RMSNorm of a one-hot vector
    assert r[0, 3] == pytest.approx(amp * c3, rel=1e-2) and r[0, 67] == pytest.approx(amp * s3, rel=1e-2)


# ---- bf16 GEMV (matmul_kernel.cu:6-63) --------------------------------------------------------------

@pytest.mark.parametrize("n,k", [(7, 8), (5, 264), (3, 2048), (4, 2560), (2, 9728)])
def test_gemv_against_float64(oracle, n, k):
    """The restated 256-thread summation order against an exact float64 product: fp32 accumulation of k
    exact products stays within k * 2^-24 of the sum of magnitudes (far inside: the tree keeps partial
    sums short), and a transposed operand or a dropped chunk would miss by orders of magnitude."""
    rng = np.random.RandomState(n * k)
    x = synth.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))
    w = synth.f32_to_bf16_bits(rng.standard_normal((n, k)).astype(np.float32))
    xf, wf = synth.bf16_bits_to_f32(x).astype(np.float64), synth.bf16_bits_to_f32(w).astype(np.float64)
    exact = wf @ xf
    got = oracle.gemv_bf16(x, w)
    assert np.all(np.abs(got - exact) <= 2e-6 * (np.abs(wf) @ np.abs(xf)))


def test_gemv_exact_sums_and_one_hot(oracle):
    k, n = 2048 + 264, 6
    rng = np.random.RandomState(1)
    w = synth.f32_to_bf16_bits(rng.standard_normal((n, k)).astype(np.float32))
    for i in (0, 9, 2047, 2048, k - 1):                       # every thread slot and the ragged last sweep
        x = np.zeros(k, dtype=np.float32)
        x[i] = 1.0
        assert np.array_equal(oracle.gemv_bf16(synth.f32_to_bf16_bits(x), w), synth.bf16_bits_to_f32(w[:, i]))
    xi = rng.randint(-8, 9, size=k).astype(np.float32)
    wi = rng.randint(-8, 9, size=(n, k)).astype(np.float32)  # integer sums are exact in any order
    got = oracle.gemv_bf16(synth.f32_to_bf16_bits(xi), synth.f32_to_bf16_bits(wi))
    assert np.array_equal(got, (wi.astype(np.float64) @ xi.astype(np.float64)).astype(np.float32))


def test_gemv_matches_torch_bf16_matmul_rounding(oracle):
    """Rounded to bf16 the result agrees with torch's fp32 matmul of the widened operands up to one step."""
    import torch
    rng = np.random.RandomState(5)
    n, k = 64, 1024
    x = synth.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))
    w = synth.f32_to_bf16_bits((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    ref = (torch.from_numpy(synth.bf16_bits_to_f32(w)) @ torch.from_numpy(synth.bf16_bits_to_f32(x))).numpy()
    got = oracle.gemv_bf16(x, w)
    assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(synth.bf16_bits_to_f32(w)) @ np.abs(synth.bf16_bits_to_f32(x)))


def test_oracle_under_sanitizers():
    """`make -C oracle asan`: every oracle function over exact-size heap buffers with AddressSanitizer + UBSan."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run(["make", "-C", os.path.join(root, "oracle"), "asan"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=600)
    assert res.returncode == 0 and "oracle asan check: ok" in res.stdout, res.stdout[-3000:]
