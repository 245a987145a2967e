"""The measurement kernels of the library (include/llmi_hip_probes.h): argument checks without a GPU, and
on a GPU that every launch shape bench.py uses runs, that the copy kernel copies and that the hand-over
probe reports what its policies are known to do."""
import ctypes

import numpy as np
import pytest

from llminfer_amd import _binding as B

P = 0x1000  # any aligned non-null address: the checks below return before anything is launched


def test_stream_read_rejects_bad_arguments():
    f = B.lib().llmi_hip_probe_stream_read
    assert f(None, P, 4096, 1, 4, 1, P, None) == B.STATUS["NULL_POINTER"]
    assert f(P, P, 4096, 1, 4, 1, None, None) == B.STATUS["NULL_POINTER"]
    assert f(P, P, 0, 1, 4, 1, P, None) == B.STATUS["INVALID_ARG"]
    assert f(P, P, 4097, 1, 4, 1, P, None) == B.STATUS["INVALID_ARG"]
    assert f(P, P, 4096, 0, 4, 1, P, None) == B.STATUS["INVALID_ARG"]
    assert f(P + 8, P, 4096, 1, 4, 1, P, None) == B.STATUS["ALIGNMENT"]


def test_stream_read_rows_rejects_bad_arguments():
    f = B.lib().llmi_hip_probe_stream_read_rows
    assert f(None, P, 64, 8, 1, 4, 1, P, None) == B.STATUS["NULL_POINTER"]
    assert f(P, P, 0, 8, 1, 4, 1, P, None) == B.STATUS["INVALID_ARG"]
    assert f(P, P, 65, 8, 1, 4, 1, P, None) == B.STATUS["INVALID_ARG"]      # rows: whole 16-row tiles
    assert f(P, P, 64, 0, 1, 4, 1, P, None) == B.STATUS["INVALID_ARG"]
    assert f(P, P, 64, 8, 5, 4, 1, P, None) == B.STATUS["INVALID_ARG"]      # more workgroups per head than tiles
    assert f(P, P + 4, 64, 8, 1, 4, 1, P, None) == B.STATUS["ALIGNMENT"]


def test_copy_and_handover_reject_bad_arguments():
    lib = B.lib()
    assert lib.llmi_hip_probe_copy(None, P, 16, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_copy(P, P, 24, None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_copy(P, P + 4, 16, None) == B.STATUS["ALIGNMENT"]
    assert lib.llmi_hip_probe_handover(0, 2, 0, 8, 0, None, None, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_block_pingpong(None, P, P, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_block_pingpong(P, P + 128, P, None) == B.STATUS["ALIGNMENT"]
    assert lib.llmi_hip_probe_placement(256, 0, None, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_placement(0, 0, P, None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_placement(4097, 0, P, None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_placement(256, 0, P + 2, None) == B.STATUS["ALIGNMENT"]
    res = B.ProbeHandoverResult()
    assert lib.llmi_hip_probe_handover(5, 2, 0, 8, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_handover(0, 2, 0, 0, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_handover(0, 2, 0, 16, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_handover(0, 2, 3, 8, 0, P + 16, ctypes.byref(res), None) == B.STATUS["ALIGNMENT"]


@pytest.fixture(scope="module")
def dev():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


@pytest.mark.gpu
def test_stream_probes_run_every_launch_shape(dev):
    """Both stream kernels over ragged tile counts (runs that differ by a tile, fewer tiles than wavefronts x tiles
    in flight): the launches succeed, the sink stays untouched, and the buffers end where the reads end."""
    import torch
    lib = B.lib()
    rows, heads = 16 * 37, 8                       # 37 tiles: no workgroup count below divides it
    nbytes = rows * heads * 256
    k = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
    v = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
    sink = torch.zeros(64, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for waves in (1, 2, 4, 8):
        for inflight in (1, 2, 4):
            for wg in (1, 3, 8, 37):
                assert lib.llmi_hip_probe_stream_read_rows(k.data_ptr(), v.data_ptr(), rows, heads, wg, waves, inflight,
                                                           sink.data_ptr(), stream) == 0
            for wg in (1, 5, 64, nbytes // 4096):
                assert lib.llmi_hip_probe_stream_read(k.data_ptr(), v.data_ptr(), nbytes, wg, waves, inflight, sink.data_ptr(),
                                                      stream) == 0
    assert lib.llmi_hip_probe_stream_read(k.data_ptr(), v.data_ptr(), nbytes, 4, 3, 1, sink.data_ptr(), stream) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_stream_read_rows(k.data_ptr(), v.data_ptr(), rows, heads, 4, 4, 3, sink.data_ptr(), stream) == B.STATUS["INVALID_ARG"]
    torch.cuda.synchronize()
    assert int(sink.abs().sum()) == 0


@pytest.mark.gpu
def test_copy_probe_copies(dev):
    import torch
    src = torch.randint(-2**31, 2**31 - 1, (1 << 20,), dtype=torch.int32, device=dev)
    dst = torch.zeros_like(src)
    assert B.lib().llmi_hip_probe_copy(src.data_ptr(), dst.data_ptr(), src.numel() * 4, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)


@pytest.mark.gpu
@pytest.mark.parametrize("reader", [8, 9])
def test_handover_probe_device_scope_sees_the_store(dev, reader):
    """A device-scope (sc1) load sees a device-scope store from another workgroup, on the writer's XCD and on the
    next one, within the bounded poll budget; the result names the XCDs both sides ran on."""
    import torch
    line = torch.zeros(4096 // 4 + 64, dtype=torch.int32, device=dev)
    base = (line.data_ptr() + 255) & ~255
    res = torch.zeros(8, dtype=torch.int32, device=dev)
    rc = B.lib().llmi_hip_probe_handover(B.PROBE_SC1, B.PROBE_SC1, 0, reader, 1, base, res.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    seen, polls, ns, xr, xw = (int(x) for x in res[:5].cpu())
    assert seen == 1 and 1 <= polls < 4000 and ns > 0
    assert 0 <= xr < 8 and 0 <= xw < 8


@pytest.mark.gpu
@pytest.mark.parametrize("exclusive", [0, 1])
def test_placement_probe_names_a_cu_for_every_workgroup(dev, exclusive):
    """One workgroup per CU is what the split path's grid counts on: 256 workgroups with a decode workgroup's LDS
    footprint report their XCD and CU; every XCD takes its share and at least half the grid has a CU of its own
    (on the boxes measured: all 256)."""
    import torch
    ids = torch.zeros(2 * 256, dtype=torch.int32, device=dev)
    assert B.lib().llmi_hip_probe_placement(256, exclusive, ids.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    a = ids.cpu().numpy().astype(np.uint32).reshape(-1, 2)
    assert np.all(a[:, 0] < 16) and np.all(a[:, 1] != 0)
    cus = {(int(x), (int(h) >> 8) & 0xFF) for x, h in a}
    assert len(cus) >= 128
    assert len(set(int(x) for x in a[:, 0])) >= 1


@pytest.mark.gpu
def test_pingpong_probe_times_both_blocks_from_every_xcd(dev):
    """Eight pairs of workgroups, each pair on one XCD, hand 64 numbers to and fro through two neighbouring 8 KiB blocks:
    every number arrives, the pairs cover both sides of the package, the times are a few hundred ns per hand-over, and
    the two sides disagree about which block is nearer (what llmi_hip_mha_workspace_side reads off)."""
    import torch
    buf = torch.zeros((64 << 10) // 4, dtype=torch.int32, device=dev)
    base = (buf.data_ptr() + 16383) & ~16383
    out = torch.zeros(64, dtype=torch.int32, device=dev)
    assert B.lib().llmi_hip_probe_block_pingpong(base, base + 8192, out.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    r = out.cpu().numpy().astype(np.int64).reshape(8, 8)
    assert np.all(r[:, 3] == 1)                                   # nothing lost
    assert np.all(r[:, 0] == r[:, 5]) and np.all(r[:, 0] < 8)     # a pair shares an XCD
    assert {int(x) >> 2 for x in r[:, 0]} == {0, 1}               # both sides of the package
    per_handover_ns = r[:, 1:3] * 10 / 64
    assert np.all(per_handover_ns > 100) and np.all(per_handover_ns < 5000)
    d = [np.mean((r[:, 1] - r[:, 2])[(r[:, 0] >> 2) == s]) for s in (0, 1)]
    assert d[0] * d[1] < 0
