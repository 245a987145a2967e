"""GPU parity of llmi_hip_gemv / llmi_hip_qkv_gemv (through the C ABI) against the CPU oracle's restatement
of the reference's bf16 GEMV kernels (matmul_kernel.cu:38-298): bf16 inputs, fp32 accumulate.

The two sides add the same exact products in a different order, so the fp32 sums agree to a few ulp of
the largest partial sum; the gate is |d| <= 4e-6 * sum_k |x_k w_k| on the fp32 result, plus half a bf16
step of the reference where the output is rounded to bf16."""
import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import to_dev

pytestmark = pytest.mark.gpu


def _case(seed, n, k):
    rng = np.random.RandomState(seed)
    x = synth.f32_to_bf16_bits(rng.standard_normal(k).astype(np.float32))
    w = synth.f32_to_bf16_bits((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    sumabs = np.abs(synth.bf16_bits_to_f32(w).astype(np.float64)) @ np.abs(synth.bf16_bits_to_f32(x).astype(np.float64))
    return x, w, sumabs


def _gate(got, ref32, sumabs, bf16_out, what):
    d = np.abs(got.astype(np.float64) - ref32.astype(np.float64))
    bound = 4e-6 * sumabs + 1e-30
    if bf16_out:
        bound = bound + np.abs(ref32) / 256.0
    assert np.all(np.isfinite(got)), what
    assert np.all(d <= bound), "%s: worst excess %.3e at row %d" % (what, (d - bound).max(), int((d - bound).argmax()))


SHAPES = [(6144, 2560), (2560, 4096), (4096, 2560), (2560, 9728), (3072, 1024), (1024, 2048), (5, 8), (17, 520),
          (33, 1032), (1, 4096), (151, 1536)]


@pytest.mark.parametrize("n,k", SHAPES)
def test_gemv_bf16_and_fp32_outputs(oracle, dev, n, k):
    x, w, sumabs = _case(n + k, n, k)
    ref = oracle.gemv_bf16(x, w)
    x_d, w_d = to_dev(x, dev), to_dev(w, dev)
    out16 = torch.full((n + 8,), 0x7FC0, dtype=torch.int16, device=dev)
    out32 = torch.full((n + 8,), float("nan"), dtype=torch.float32, device=dev)
    ops.gemv(x_d, w_d, out16[:n], mode=B.GEMV_OUT_BF16)
    ops.gemv(x_d, w_d, out32[:n], mode=B.GEMV_OUT_F32)
    torch.cuda.synchronize()
    got32 = out32.cpu().numpy()
    got16 = out16.cpu().numpy().view(np.uint16)
    _gate(got32[:n], ref, sumabs, False, "fp32 output %dx%d" % (n, k))
    _gate(synth.bf16_bits_to_f32(got16[:n]), ref, sumabs, True, "bf16 output %dx%d" % (n, k))
    assert np.all(np.isnan(got32[n:])) and np.all(got16[n:] == 0x7FC0)  # nothing written past row n
    # the bf16 output is the rounding of the kernel's own fp32 sum
    assert np.array_equal(got16[:n], synth.f32_to_bf16_bits(got32[:n]))


@pytest.mark.parametrize("n,k", [(2560, 4096), (1024, 2048), (19, 264)])
def test_gemv_with_residual_add(oracle, dev, n, k):
    """fused_gemv_add: residual[r] = bf16(float(residual[r]) + sum) (matmul_kernel.cu:167-171)."""
    x, w, sumabs = _case(3 * n + k, n, k)
    rng = np.random.RandomState(n)
    res = synth.f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32))
    ref = synth.bf16_bits_to_f32(res) + oracle.gemv_bf16(x, w)
    res_d = to_dev(res.copy(), dev)
    ops.gemv(to_dev(x, dev), to_dev(w, dev), res_d, mode=B.GEMV_ADD_BF16)
    torch.cuda.synchronize()
    _gate(synth.bf16_bits_to_f32(res_d.cpu().numpy().view(np.uint16)), ref.astype(np.float32), sumabs, True,
          "residual add %dx%d" % (n, k))


@pytest.mark.parametrize("dim,kv_dim,k", [(4096, 1024, 2560), (2048, 1024, 1024), (8192, 1024, 5120), (384, 128, 264)])
def test_packed_qkv_gemv(oracle, dev, dim, kv_dim, k):
    n = dim + 2 * kv_dim
    x, w, sumabs = _case(dim + k, n, k)
    ref = oracle.gemv_bf16(x, w)
    q = torch.zeros(dim, dtype=torch.int16, device=dev)
    kk = torch.zeros(kv_dim, dtype=torch.int16, device=dev)
    v = torch.zeros(kv_dim, dtype=torch.int16, device=dev)
    ops.qkv_gemv(to_dev(x, dev), to_dev(w, dev), q, kk, v)
    torch.cuda.synchronize()
    got = np.concatenate([t.cpu().numpy().view(np.uint16) for t in (q, kk, v)])
    _gate(synth.bf16_bits_to_f32(got), ref, sumabs, True, "packed qkv %d+2*%d x %d" % (dim, kv_dim, k))


def test_gemv_exact_cases(dev):
    """Sums that are exact in fp32 must come out exactly, whatever the order: one-hot inputs pick a weight
    column, small integers add up without rounding."""
    n, k = 70, 1024
    rng = np.random.RandomState(0)
    w = synth.f32_to_bf16_bits(rng.standard_normal((n, k)).astype(np.float32))
    out = torch.zeros(n, dtype=torch.float32, device=dev)
    for i in (0, 7, 8, 511, 512, 1023):
        x = np.zeros(k, dtype=np.float32)
        x[i] = 1.0
        ops.gemv(to_dev(synth.f32_to_bf16_bits(x), dev), to_dev(w, dev), out, mode=B.GEMV_OUT_F32)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), synth.bf16_bits_to_f32(w[:, i]))
    xi = rng.randint(-8, 9, size=k).astype(np.float32)
    wi = rng.randint(-8, 9, size=(n, k)).astype(np.float32)
    ops.gemv(to_dev(synth.f32_to_bf16_bits(xi), dev), to_dev(synth.f32_to_bf16_bits(wi), dev), out, mode=B.GEMV_OUT_F32)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), (wi.astype(np.float64) @ xi.astype(np.float64)).astype(np.float32))
