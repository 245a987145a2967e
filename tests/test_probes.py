"""The measurement kernels of the library (include/llmi_hip_probes.h) and the diagnostic probes of libllmi_diag.so
(include/llmi_hip_diag.h): argument checks without a GPU, and on a GPU that every launch shape bench.py uses runs,
that the copy kernel copies and that the probes report what they are documented to report. Timings are printed,
never asserted: they depend on the box."""
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


def test_stream_tiles_rejects_bad_arguments():
    f = B.lib().llmi_hip_probe_stream_tiles
    ok = dict(positions=64, kv_heads=8, kv_layout=1, splits=2, waves=4, inflight=2, mode=2, pause=0, stagger=0)

    def call(k=P, v=P, sink=P, **over):
        a = dict(ok, **over)
        return f(k, v, a["positions"], a["kv_heads"], a["kv_layout"], a["splits"], a["waves"], a["inflight"], a["mode"], a["pause"],
                 a["stagger"], sink, None)

    assert call(k=None) == B.STATUS["NULL_POINTER"] and call(sink=None) == B.STATUS["NULL_POINTER"]
    assert call(positions=0) == B.STATUS["INVALID_ARG"] and call(positions=65) == B.STATUS["INVALID_ARG"]
    assert call(splits=5) == B.STATUS["INVALID_ARG"]        # more splits than tiles
    assert call(kv_layout=2) == B.STATUS["LAYOUT"]
    assert call(mode=4) == B.STATUS["INVALID_ARG"] and call(pause=-1) == B.STATUS["INVALID_ARG"]
    assert call(stagger=-1) == B.STATUS["INVALID_ARG"] and call(stagger=256) == B.STATUS["INVALID_ARG"]
    assert call(k=P + 8) == B.STATUS["ALIGNMENT"]


def test_copy_and_handover_reject_bad_arguments():
    lib = B.lib()
    assert lib.llmi_hip_probe_copy(None, P, 16, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_copy(P, P, 24, None) == B.STATUS["INVALID_ARG"]
    assert lib.llmi_hip_probe_copy(P, P + 4, 16, None) == B.STATUS["ALIGNMENT"]
    assert lib.llmi_hip_probe_block_pingpong(None, P, P, None) == B.STATUS["NULL_POINTER"]
    assert lib.llmi_hip_probe_block_pingpong(P, P + 128, P, None) == B.STATUS["ALIGNMENT"]
    diag = B.diag_lib()
    assert diag.llmi_diag_handover(0, 2, 0, 8, 0, None, None, None) == B.STATUS["NULL_POINTER"]
    assert diag.llmi_diag_placement(256, 0, None, None) == B.STATUS["NULL_POINTER"]
    assert diag.llmi_diag_placement(0, 0, P, None) == B.STATUS["INVALID_ARG"]
    assert diag.llmi_diag_placement(4097, 0, P, None) == B.STATUS["INVALID_ARG"]
    assert diag.llmi_diag_placement(256, 0, P + 2, None) == B.STATUS["ALIGNMENT"]
    res = B.DiagHandoverResult()
    assert diag.llmi_diag_handover(5, 2, 0, 8, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert diag.llmi_diag_handover(0, 2, 0, 0, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert diag.llmi_diag_handover(0, 2, 0, 16, 0, P, ctypes.byref(res), None) == B.STATUS["INVALID_ARG"]
    assert diag.llmi_diag_handover(0, 2, 3, 8, 0, P + 16, ctypes.byref(res), None) == B.STATUS["ALIGNMENT"]


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
def test_stream_tiles_probe_runs_every_mode_and_shape(dev):
    """Every mode, launch shape and layout of the stream-variants kernel on ragged tile counts: the launches succeed, the
    sink stays untouched, and an unsupported (waves, tiles in flight) pair is refused."""
    import torch
    lib = B.lib()
    positions, heads = 16 * 37, 8
    nbytes = positions * heads * 256
    k = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
    v = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
    sink = torch.zeros(64, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for layout in (0, 1):
        for waves, inflight in ((4, 2), (8, 1), (8, 2), (4, 4)):
            for mode in range(4):
                for splits in (1, 3, 8, 37):
                    for stagger in (0, 1, 2, 4 * 31, 2 + 4 * 7):  # none, mask 3, split-fastest grid, mask 31, both
                        assert lib.llmi_hip_probe_stream_tiles(k.data_ptr(), v.data_ptr(), positions, heads, layout, splits, waves, inflight,
                                                               mode, 2, stagger, sink.data_ptr(), stream) == 0
    assert lib.llmi_hip_probe_stream_tiles(k.data_ptr(), v.data_ptr(), positions, heads, 1, 4, 2, 2, 0, 0, 0, sink.data_ptr(),
                                           stream) == B.STATUS["INVALID_ARG"]
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
    rc = B.diag_lib().llmi_diag_handover(B.DIAG_SC1, B.DIAG_SC1, 0, reader, 1, base, res.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    seen, polls, ns, xr, xw = (int(x) for x in res[:5].cpu())
    assert seen == 1 and 1 <= polls < 4000 and ns > 0
    assert 0 <= xr < 8 and 0 <= xw < 8


@pytest.mark.gpu
@pytest.mark.parametrize("exclusive", [0, 1])
def test_placement_probe_names_a_cu_for_every_workgroup(dev, exclusive):
    """256 workgroups with a decode workgroup's LDS footprint report their XCD and CU (on the boxes measured: 256
    different CUs, 32 per XCD; printed, not asserted: the split path does not rely on it for its result)."""
    import torch
    ids = torch.zeros(2 * 256, dtype=torch.int32, device=dev)
    assert B.diag_lib().llmi_diag_placement(256, exclusive, ids.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    a = ids.cpu().numpy().astype(np.uint32).reshape(-1, 2)
    assert np.all(a[:, 0] < 16) and np.all(a[:, 1] != 0)
    cus = {(int(x), (int(h) >> 8) & 0xFF) for x, h in a}
    print("placement: %d distinct CUs, %d XCDs for 256 workgroups" % (len(cus), len(set(int(x) for x in a[:, 0]))))


@pytest.mark.gpu
def test_pingpong_probe_times_both_blocks_from_every_xcd(dev):
    """Eight pairs of workgroups, each pair on one XCD, hand 64 numbers to and fro through two neighbouring 8 KiB blocks:
    every number arrives and every workgroup names the XCD it ran on (pairs share one when workgroups are dealt to the
    XCDs in turn; a pair that did not is left out of the decision). The times (a few hundred ns per hand-over on the boxes measured,
    the two sides of the package disagreeing about which block is nearer) are what llmi_hip_mha_workspace_side reads
    off; they are printed here, the decision taken from them is tested with made-up timings on the CPU."""
    import torch
    buf = torch.zeros((64 << 10) // 4, dtype=torch.int32, device=dev)
    base = (buf.data_ptr() + 16383) & ~16383
    out = torch.zeros(64, dtype=torch.int32, device=dev)
    assert B.lib().llmi_hip_probe_block_pingpong(base, base + 8192, out.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    r = out.cpu().numpy().astype(np.int64).reshape(8, 8)
    assert np.all(r[:, 3] == 1)                                   # nothing lost
    assert np.all(r[:, 0] < 8) and np.all(r[:, 5] < 8)            # both workgroups of a pair name their XCD
    assert np.all(r[:, 1:3] > 0)
    per_handover_ns = r[:, 1:3] * 10 / 64
    d = [np.mean((r[:, 1] - r[:, 2])[(r[:, 0] >> 2) == s]) if np.any((r[:, 0] >> 2) == s) else float("nan") for s in (0, 1)]
    print("ping-pong: %d of 8 pairs on one XCD; %.0f .. %.0f ns per hand-over; clear minus set block, ticks: XCDs 0-3 %+.0f, XCDs 4-7 %+.0f; decision %d"
          % (int(np.sum(r[:, 0] == r[:, 5])), per_handover_ns.min(), per_handover_ns.max(), d[0], d[1],
             B.lib().llmi_hip_side_from_pingpong(out.cpu().numpy().astype(np.uint32).ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)))))
