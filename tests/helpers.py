"""Shared helpers of the GPU parity tests: upload a synthetic case, run it
through the C ABI, compare with the CPU oracle."""
import numpy as np
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

# Tolerance of the parity gate: bf16 inputs, fp32 accumulate.
ATOL = 2e-3
RTOL = 1e-2


def to_dev(a_u16, dev):
    """uint16 numpy bit patterns -> device tensor (int16 view carries the same bits)."""
    return torch.from_numpy(a_u16.view(np.int16)).to(dev)


def from_dev_bf16(t):
    return synth.bf16_bits_to_f32(t.cpu().numpy().view(np.uint16))


def run_hip(case, dev, *, kv_layout=B.KV_LAYOUT_POS_MAJOR, force_path=B.PATH_AUTO, num_splits=0,
            waves_per_group=0, workspace_bytes=None, want_plan=False, workspace_side=0, workspace_offset=0):
    """Runs llmi_hip_mha_decode on a case from synth.make_case. Returns (bf16 out as f32, f32 tap[, plan])."""
    n_kv = case["kv_dim"] // case["head_dim"]
    k, v = case["k"], case["v"]
    if kv_layout == B.KV_LAYOUT_HEAD_MAJOR:
        k = synth.to_head_major(k, n_kv)
        v = synth.to_head_major(v, n_kv)
    q_d, k_d, v_d = to_dev(case["q"], dev), to_dev(k, dev), to_dev(v, dev)
    out = torch.full((case["head_num"] * case["head_dim"],), 0x7FC0, dtype=torch.int16, device=dev)
    out32 = torch.full((case["head_num"] * case["head_dim"],), float("nan"), dtype=torch.float32, device=dev)
    if workspace_bytes is None:
        workspace_bytes = ops.workspace_bytes(case["head_num"], case["head_dim"], case["max_seq_len"])
    ws = torch.full((max(workspace_bytes // 4, 4) + workspace_offset // 4,), float("nan"), dtype=torch.float32, device=dev)
    ws = ws[workspace_offset // 4:]
    if workspace_side == "measure":  # what an engine does once per workspace; the measurement overwrites part of it
        # (a measurement that makes no statement is replaced by a claim: the side word only ever changes the time)
        workspace_side = ops.workspace_side(ws) or 0x55555555
        ws.fill_(float("nan"))
    scal = dict(layer_id=case["layer_id"], pos=case["pos"], kv_dim=case["kv_dim"], kv_mul=case["kv_mul"],
                head_num=case["head_num"], head_dim=case["head_dim"], max_seq_len=case["max_seq_len"],
                kv_layout=kv_layout, force_path=force_path, num_splits=num_splits,
                waves_per_group=waves_per_group, workspace_side=workspace_side)
    plan = ops.mha_plan(ops.make_mha_args(q_d, k_d, v_d, out, ws, **scal))
    ops.mha_decode(q_d, k_d, v_d, out, ws, output_f32=out32, **scal)
    torch.cuda.synchronize()
    res = (from_dev_bf16(out), out32.cpu().numpy())
    return res + (plan,) if want_plan else res


def run_oracle(oracle, case):
    return oracle.mha_cpu(case["q"], case["k"], case["v"], case["layer_id"], case["pos"], case["kv_dim"],
                          case["kv_mul"], case["head_num"], case["head_dim"], case["max_seq_len"])


def parity_report(got, ref):
    d = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    max_abs = float(d.max())
    max_rel = float((d / np.maximum(np.abs(ref), 1e-30)).max())
    ok = bool(np.all(d <= ATOL + RTOL * np.abs(ref))) and bool(np.all(np.isfinite(got)))
    return ok, max_abs, max_rel


def assert_parity(got, ref, what=""):
    """The gate on the bf16 output: |d| <= ATOL + RTOL*|ref| elementwise. (A bare max-abs of 2e-3 cannot
    hold on a bf16 output of magnitude ~1, whose rounding step alone is 2^-8; the bare max-abs and
    max-rel bounds are asserted on the fp32 tap instead, see assert_tap_parity.)"""
    ok, max_abs, max_rel = parity_report(got, ref)
    assert ok, "%s: max_abs=%.3e max_rel=%.3e exceeds |d| <= %g + %g*|ref|" % (what, max_abs, max_rel, ATOL, RTOL)
    return max_abs, max_rel


def assert_tap_parity(got32, ref, what=""):
    """fp32 tap (result before bf16 rounding): max-abs <= 2e-3 and max-rel <= 1e-2 separately (max-rel over
    elements that are not vanishingly small), plus a tight bound that leaves room only for summation
    order and the hardware exp2."""
    d = np.abs(got32.astype(np.float64) - ref.astype(np.float64))
    assert np.all(np.isfinite(got32)), what
    assert d.max() <= ATOL, "%s: fp32 tap max_abs=%.3e > %g" % (what, d.max(), ATOL)
    big = np.abs(ref) > 1e-4
    if big.any():
        rel = (d[big] / np.abs(ref[big])).max()
        assert rel <= RTOL, "%s: fp32 tap max_rel=%.3e > %g" % (what, rel, RTOL)
    assert np.all(d <= 2e-5 + 2e-4 * np.abs(ref)), "%s: fp32 tap max_abs=%.3e beyond round-off" % (what, d.max())
