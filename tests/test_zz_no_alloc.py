"""llmi_hip_mha_decode_static (the entry point that allocates nothing: its split workspace is a fixed
array inside the library's code object) against llmi_hip_mha_decode through the C ABI: same inputs, same
plan, so the same bits; two calls in a row, the second on a smaller input, both also against the oracle."""
import ctypes

import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import assert_parity, from_dev_bf16, run_oracle, to_dev

pytestmark = pytest.mark.gpu

STATIC_BYTES = 4 << 20


def _run_both(case, dev, poison, warm, **over):
    n_kv = case["kv_dim"] // case["head_dim"]
    q = to_dev(case["q"], dev)
    k = to_dev(synth.to_head_major(case["k"], n_kv), dev)
    v = to_dev(synth.to_head_major(case["v"], n_kv), dev)
    n = case["head_num"] * case["head_dim"]
    ws = torch.full((STATIC_BYTES // 4,), float("nan"), dtype=torch.float32, device=dev)  # same size as the static array
    bufs = {e: (torch.full((n,), poison, dtype=torch.int16, device=dev),
                torch.full((n,), float("nan"), dtype=torch.float32, device=dev))
            for e in ("llmi_hip_mha_decode", "llmi_hip_mha_decode_static")}
    outs = []
    free_before = None
    for entry, (out, out32) in bufs.items():
        a = ops.make_mha_args(q, k, v, out, ws if entry == "llmi_hip_mha_decode" else None, layer_id=case["layer_id"],
                              pos=case["pos"], kv_dim=case["kv_dim"], kv_mul=case["kv_mul"], head_num=case["head_num"],
                              head_dim=case["head_dim"], max_seq_len=case["max_seq_len"],
                              kv_layout=B.KV_LAYOUT_HEAD_MAJOR, output_f32=out32, **over)
        if entry == "llmi_hip_mha_decode_static" and warm:
            free_before = torch.cuda.mem_get_info(dev)[0]
        B.check(getattr(B.lib(), entry)(ctypes.byref(a)), entry)
        torch.cuda.synchronize()
        if free_before is not None:  # the device's free memory is what it was: nothing was allocated
            assert torch.cuda.mem_get_info(dev)[0] == free_before
        outs.append((out.cpu().numpy().view(np.uint16), out32.cpu().numpy()))
    return outs


def test_static_workspace_entry_point_matches_the_allocating_one(oracle, dev):
    warm = False  # the first call on a device looks the array's address up; from then on free memory must not move
    # first a long context (32 splits), then a shorter one with fewer splits and fewer heads on the same
    # static array, which still holds the first call's partial results and records; then single pass
    for seed, ctx, n_q, n_kv, poison in ((41, 6000, 32, 8, 0x7FC0), (42, 700, 16, 8, 0x7FC1), (43, 90, 32, 8, 0x7FC0)):
        case = synth.make_case(seed, ctx=ctx, n_q=n_q, n_kv=n_kv)
        (ref_bits, ref32), (got_bits, got32) = _run_both(case, dev, poison, warm)
        warm = True
        assert np.array_equal(got_bits, ref_bits), "ctx %d: bf16 outputs differ" % ctx
        assert np.array_equal(got32, ref32), "ctx %d: fp32 taps differ" % ctx
        assert_parity(synth.bf16_bits_to_f32(got_bits), run_oracle(oracle, case), "static entry point, ctx %d" % ctx)


def test_static_workspace_entry_point_rejects_what_does_not_fit(dev):
    case = synth.make_case(44, ctx=5000, n_q=64, n_kv=8)
    dummy = torch.zeros(64 * 128, dtype=torch.int16, device=dev)
    a = ops.make_mha_args(dummy, dummy, dummy, dummy, None, layer_id=0, pos=case["pos"], kv_dim=1024, kv_mul=8,
                          head_num=64, head_dim=128, max_seq_len=case["max_seq_len"], kv_layout=B.KV_LAYOUT_HEAD_MAJOR,
                          force_path=B.PATH_SPLIT_FUSED, num_splits=256)  # 64 * 256 * 528 bytes > 4 MiB
    assert B.lib().llmi_hip_mha_decode_static(ctypes.byref(a)) == B.STATUS["WORKSPACE"]
    assert b"static workspace" in B.lib().llmi_hip_last_error()
    assert B.lib().llmi_hip_mha_decode_static(None) == B.STATUS["NULL_POINTER"]
    # the automatic plan takes what fits instead: 64 heads x 32 splits is well inside
    a.force_path, a.num_splits = B.PATH_AUTO, 0
    plan = ops.mha_plan(ops.make_mha_args(dummy, dummy, dummy, dummy, torch.empty(STATIC_BYTES // 4, device=dev), layer_id=0,
                                          pos=case["pos"], kv_dim=1024, kv_mul=8, head_num=64, head_dim=128,
                                          max_seq_len=case["max_seq_len"], kv_layout=B.KV_LAYOUT_HEAD_MAJOR))
    assert plan.workspace_needed <= STATIC_BYTES
