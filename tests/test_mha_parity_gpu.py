"""GPU parity of llmi_hip_mha_decode (through the C ABI) against the CPU oracle
on the same seeded, bf16-rounded inputs. Gate: |d| <= 2e-3 + 1e-2*|ref| on the
bf16 output, and max-abs <= 2e-3; the fp32 tap is held to a tighter bound."""
import ctypes

import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import assert_parity, assert_tap_parity, run_hip, run_oracle

pytestmark = pytest.mark.gpu

QWEN3_4B = dict(n_q=32, n_kv=8)


def _check(oracle, dev, case, **kw):
    ref = run_oracle(oracle, case)
    got16, got32, plan = run_hip(case, dev, want_plan=True, **kw)
    what = "ctx=%d path=%d splits=%d waves=%d %s" % (case["pos"] + 1, plan.path, plan.num_splits,
                                                     plan.waves_per_group, kw)
    assert_parity(got16, ref, "bf16 out " + what)
    assert_tap_parity(got32, ref, what)
    return plan


@pytest.mark.parametrize("ctx", [128, 512, 1024, 2048])
@pytest.mark.parametrize("layout", [B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])
def test_qwen3_4b_short_context(oracle, dev, ctx, layout):
    """Qwen3-4B layer shape, ctx 128..2048, seed 2, both cache layouts, dispatcher's choice."""
    case = synth.make_case(2, ctx=ctx, **QWEN3_4B)
    _check(oracle, dev, case, kv_layout=layout)


@pytest.mark.parametrize("ctx", [128, 512, 1024, 2048])
def test_single_pass_forced(oracle, dev, ctx):
    case = synth.make_case(2, ctx=ctx, **QWEN3_4B)
    plan = _check(oracle, dev, case, force_path=B.PATH_SINGLE_PASS)
    assert plan.path == B.PATH_SINGLE_PASS and plan.num_splits == 1


@pytest.mark.parametrize("ctx", [4096, 8192, 16384, 32768])
def test_qwen3_4b_long_context(oracle, dev, ctx):
    """Long-context KV-split path, seed 3, head-major layout (the production layout)."""
    case = synth.make_case(3, ctx=ctx, **QWEN3_4B)
    plan = _check(oracle, dev, case, kv_layout=B.KV_LAYOUT_HEAD_MAJOR)
    assert plan.path == B.PATH_SPLIT_FUSED and plan.num_splits > 1


@pytest.mark.parametrize("splits", [2, 4, 8, 16, 32, 64, 256])
@pytest.mark.parametrize("waves", [1, 2, 4, 8])
@pytest.mark.parametrize("path", [B.PATH_SPLIT, B.PATH_SPLIT_FUSED])
def test_split_sweep_matches_oracle(oracle, dev, splits, waves, path):
    """Any split count / workgroup shape gives the oracle's answer (ctx 4096), with the separate
    combine kernel and with the combine fused into the split kernel's last-arriving workgroup."""
    case = synth.make_case(3, ctx=4096, **QWEN3_4B)
    _check(oracle, dev, case, num_splits=splits, waves_per_group=waves, force_path=path)


_LONG_REF = {}


@pytest.mark.parametrize("splits", [4, 8, 16, 32, 64])
@pytest.mark.parametrize("ctx", [8192, 16384, 32768])
def test_split_sweep_long_context_matches_oracle(oracle, dev, ctx, splits):
    """The long-context configuration at its full sizes: split counts 4 .. 64 at ctx 8192, 16384 and 32768
    against the oracle (fused combine, 4 waves, head-major; the oracle runs once per context length)."""
    case = synth.make_case(3, ctx=ctx, **QWEN3_4B)
    if ctx not in _LONG_REF:
        _LONG_REF[ctx] = run_oracle(oracle, case)
    ref = _LONG_REF[ctx]
    got16, got32, plan = run_hip(case, dev, want_plan=True, kv_layout=B.KV_LAYOUT_HEAD_MAJOR, force_path=B.PATH_SPLIT_FUSED,
                                 num_splits=splits, waves_per_group=4)
    assert plan.num_splits == splits and plan.path == B.PATH_SPLIT_FUSED
    what = "ctx=%d splits=%d" % (ctx, splits)
    assert_parity(got16, ref, "bf16 out " + what)
    assert_tap_parity(got32, ref, what)


@pytest.mark.parametrize("ctx", [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 159, 160, 161, 175, 176, 177, 207, 208, 209, 239, 240, 241, 255, 256, 257, 287, 288, 289, 1000, 4097])
@pytest.mark.parametrize("path", [B.PATH_SINGLE_PASS, B.PATH_SPLIT, B.PATH_SPLIT_FUSED])
def test_ragged_lengths(oracle, dev, ctx, path):
    """Lengths around the 16-row tile, the wave count and the dispatch threshold; the cache rows past
    pos hold NaN patterns, so any over-read shows."""
    case = synth.make_case(100 + ctx, ctx=ctx, max_seq_len=ctx + 7, **QWEN3_4B)
    _check(oracle, dev, case, force_path=path, num_splits=0 if path == B.PATH_SINGLE_PASS else 5)


@pytest.mark.parametrize("n_q,n_kv", [(8, 8), (16, 8), (32, 8), (64, 8), (6, 2), (12, 4), (16, 1), (20, 4)])
@pytest.mark.parametrize("layout", [B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])
def test_group_sizes_and_layers(oracle, dev, n_q, n_kv, layout):
    """kv_mul 1..16 (incl. non powers of two), a non-zero layer of a multi-layer cache with
    max_seq_len > seq_len: the shapes of the reference's own op test (test_op_mha.cpp:9-18,68-78)."""
    case = synth.make_case(7, n_q=n_q, n_kv=n_kv, ctx=333, max_seq_len=400, layers=3, layer_id=2)
    _check(oracle, dev, case, kv_layout=layout)
    _check(oracle, dev, case, kv_layout=layout, force_path=B.PATH_SPLIT, num_splits=7)
    _check(oracle, dev, case, kv_layout=layout, force_path=B.PATH_SPLIT_FUSED, num_splits=7)


def test_unnormalised_inputs(oracle, dev):
    """Plain N(0,1) inputs (no RMS normalisation): larger score spread, peaked softmax."""
    case = synth.make_case(11, ctx=777, rms_norm=False, **QWEN3_4B)
    case["q"] = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(case["q"]) * 3.0)
    _check(oracle, dev, case)
    _check(oracle, dev, case, force_path=B.PATH_SPLIT, num_splits=13)


def test_qwen3_0p6b_layout_bf16(oracle, dev):
    """16 Q / 8 KV heads, 256 cached + 1 new position (the CPU-plumbing shape, here in bf16)."""
    case = synth.make_case(1, n_q=16, n_kv=8, ctx=257, max_seq_len=512, rms_norm=False)
    _check(oracle, dev, case)


def test_split_equals_single_pass(dev):
    """Property at full size: split and single-pass agree on the fp32 tap (ctx 32768), no oracle needed."""
    case = synth.make_case(5, ctx=32768, **QWEN3_4B)
    _, one = run_hip(case, dev, force_path=B.PATH_SINGLE_PASS)
    for path in (B.PATH_SPLIT, B.PATH_SPLIT_FUSED):
        for splits in (4, 64, 256):
            _, many = run_hip(case, dev, force_path=path, num_splits=splits)
            assert np.all(np.abs(one - many) <= 1e-5 + 1e-4 * np.abs(one))


def test_one_hot_attention(dev):
    """One key far above the rest: the output is that position's V row exactly (bf16 values pass through)."""
    case = synth.make_case(9, ctx=2000, **QWEN3_4B)
    q = synth.bf16_bits_to_f32(case["q"]).reshape(32, 128)
    k = case["k"]
    target = 1234
    for kvh in range(8):
        # K[target] = 40 * mean of the group's queries: score ~ 40*|q|^2/sqrt(128) >> all others.
        k[0, target, kvh * 128:(kvh + 1) * 128] = synth.f32_to_bf16_bits(40.0 * q[kvh * 4:(kvh + 1) * 4].mean(0))
    got16, _ = run_hip(case, dev, force_path=B.PATH_SPLIT, num_splits=16)
    want = synth.bf16_bits_to_f32(case["v"][0, target]).reshape(8, 1, 128).repeat(4, axis=1).reshape(-1)
    assert np.allclose(got16, want, atol=2e-3, rtol=1e-2)


def test_fused_combine_repeated_calls_share_workspace(oracle, dev):
    """The arrival cells of the fused combine need no clearing: back-to-back calls on one workspace
    (first full of NaN patterns), with different split counts and contexts, all match the oracle."""
    import torch
    from llminfer_amd import ops
    from helpers import from_dev_bf16, to_dev
    ws = torch.full((ops.workspace_bytes(32, 128, 4096) // 4,), float("nan"), dtype=torch.float32, device=dev)
    for seed, ctx, splits in [(21, 4096, 64), (22, 3000, 64), (23, 4096, 17), (24, 700, 0), (25, 4096, 64)]:
        case = synth.make_case(seed, ctx=ctx, max_seq_len=4096, **QWEN3_4B)
        ref = run_oracle(oracle, case)
        q, k, v = to_dev(case["q"], dev), to_dev(case["k"], dev), to_dev(case["v"], dev)
        out = torch.zeros(32 * 128, dtype=torch.int16, device=dev)
        for _ in range(3):
            ops.mha_decode(q, k, v, out, ws, layer_id=0, pos=ctx - 1, kv_dim=1024, kv_mul=4, head_num=32,
                           head_dim=128, max_seq_len=4096, force_path=B.PATH_SPLIT_FUSED, num_splits=splits)
        torch.cuda.synchronize()
        assert_parity(from_dev_bf16(out), ref, "ctx=%d splits=%d" % (ctx, splits))


def test_graph_replay_matches_eager(oracle, dev):
    """A captured decode call (fused combine) replayed several times, with eager work and
    synchronisation between the replays, gives the eager result every time."""
    import torch
    from llminfer_amd import ops
    from helpers import from_dev_bf16, to_dev
    case = synth.make_case(31, ctx=5000, **QWEN3_4B)
    ref = run_oracle(oracle, case)
    q, k, v = to_dev(case["q"], dev), to_dev(case["k"], dev), to_dev(case["v"], dev)
    ws = torch.full((ops.workspace_bytes(32, 128, 5000) // 4,), float("nan"), dtype=torch.float32, device=dev)
    out = torch.zeros(32 * 128, dtype=torch.int16, device=dev)
    kw = dict(layer_id=0, pos=4999, kv_dim=1024, kv_mul=4, head_num=32, head_dim=128, max_seq_len=5000)
    ops.mha_decode(q, k, v, out, ws, **kw)
    torch.cuda.synchronize()
    eager = out.clone()
    assert_parity(from_dev_bf16(eager), ref, "eager")
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.mha_decode(q, k, v, out, ws, stream=side, **kw)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(4):
        out.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        scratch = torch.randn(1 << 16, device=dev).sum().item()  # unrelated eager work between replays
        assert scratch == scratch


def test_fused_combine_many_calls_agree_with_the_two_launch_path(dev):
    """400 back-to-back calls on one workspace, the context, the split count and the query changing from
    call to call (some enqueued without a synchronisation in between): the fused combine -- whose splits hand
    their results over through device memory inside one launch -- must give what the split kernel followed by
    the separate combine kernel gives, up to the rounding of a different summation order."""
    import torch
    from llminfer_amd import ops
    from helpers import from_dev_bf16, to_dev
    n_q, n_kv, msl = 32, 8, 6000
    case = synth.make_case(91, ctx=msl, max_seq_len=msl, **QWEN3_4B)
    k = to_dev(synth.to_head_major(case["k"], n_kv), dev)
    v = to_dev(synth.to_head_major(case["v"], n_kv), dev)
    ws = torch.full((ops.workspace_bytes(n_q, 128, msl) // 4,), float("nan"), dtype=torch.float32, device=dev)
    ws2 = torch.zeros_like(ws)
    rng = np.random.RandomState(3)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    outs, refs = [], []
    for it in range(400):
        ctx = int(rng.choice([209, 300, 777, 1024, 2048, 3001, 4096, 5999]))
        splits = int(rng.choice([0, 0, 2, 5, 16, 31, 32, 64]))
        q = torch.randn(n_q * 128, generator=gen, device=dev).to(torch.bfloat16)
        kw = dict(layer_id=0, pos=ctx - 1, kv_dim=1024, kv_mul=4, head_num=n_q, head_dim=128, max_seq_len=msl,
                  kv_layout=B.KV_LAYOUT_HEAD_MAJOR, num_splits=splits)
        out = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        ref = torch.zeros(n_q * 128, dtype=torch.int16, device=dev)
        ops.mha_decode(q, k, v, out, ws, force_path=B.PATH_SPLIT_FUSED, **kw)
        ops.mha_decode(q, k, v, ref, ws2, force_path=B.PATH_SPLIT, **kw)
        outs.append(out)
        refs.append(ref)
        if it % 7 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    for it, (out, ref) in enumerate(zip(outs, refs)):
        g, r = from_dev_bf16(out), from_dev_bf16(ref)
        assert np.all(np.isfinite(g)), "call %d" % it
        assert np.all(np.abs(g - r) <= np.abs(r) / 128 + 1e-6), "call %d: max diff %g" % (it, np.abs(g - r).max())


@pytest.mark.parametrize("kv_mul,n_kv", [(4, 8), (16, 2)])
def test_fused_combine_gives_up_with_nan_instead_of_hanging(oracle, dev, kv_mul, n_kv):
    """The merging workgroup's wait for the other splits is bounded. With the limit forced to zero
    polls from the host every fused launch gives up at once: the kernel still ends normally and
    every output is NaN (never a plausible wrong number). With the limit restored the same call
    on the same data gives the oracle's answer. Both merge variants (one wavefront per head, and
    heads shared out when a group has more heads than the workgroup has wavefronts)."""
    case = synth.make_case(31, ctx=1000, n_q=kv_mul * n_kv, n_kv=n_kv)

    def timeouts():
        n = ctypes.c_uint64()
        assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(n)) == 0
        return n.value

    before = timeouts()
    prev = B.lib().llmi_hip_set_poll_limit(0)
    try:
        assert prev == 1 << 22
        got16, got32 = run_hip(case, dev, force_path=B.PATH_SPLIT_FUSED, num_splits=8)
    finally:
        assert B.lib().llmi_hip_set_poll_limit(prev) == 0
    assert np.all(np.isnan(got16)) and np.all(np.isnan(got32))
    # every give-up is counted on the device, one per query head, where the host can read it
    assert timeouts() == before + kv_mul * n_kv
    _check(oracle, dev, case, force_path=B.PATH_SPLIT_FUSED, num_splits=8)
    assert timeouts() == before + kv_mul * n_kv  # a call that completes counts nothing


@pytest.mark.parametrize("ctx,splits,waves", [(8192, 0, 0), (5000, 7, 4), (1000, 3, 1), (3001, 5, 2)])
def test_position_major_staggered_walk(oracle, dev, ctx, splits, waves):
    """Position-major layout, several tiles per wavefront: every split starts its walk at a different
    tile of its run and wraps round (ragged last tiles included); the result is the oracle's."""
    case = synth.make_case(23, ctx=ctx, **QWEN3_4B)
    kw = dict(force_path=B.PATH_SPLIT_FUSED, num_splits=splits, waves_per_group=waves) if splits else {}
    plan = _check(oracle, dev, case, kv_layout=B.KV_LAYOUT_POS_MAJOR, **kw)
    tiles = (ctx + 15) // 16
    assert plan.num_splits > 1 and tiles // plan.num_splits >= 2 * plan.waves_per_group  # two or more tiles per wave


def test_head_major_staggered_walk_forced(dev):
    """The staggered walk of the head-major layout, which the launcher's rule only picks from 1 MiB runs on, forced on
    small shapes (LLMI_HIP_STAGGER_MASK is read once per process: a child process): ragged runs, one to eight
    wavefronts, more rotation than a wavefront has tiles, the append variant, by-side and plain workspace; every
    result is the oracle's."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
        "import torch, oracle\n"
        "from llminfer_amd import _binding as B, synth\n"
        "from helpers import assert_parity, assert_tap_parity, run_hip, run_oracle\n"
        "oracle.lib(); dev = torch.device('cuda:0')\n"
        "assert B.lib().llmi_hip_stagger_mask(B.KV_LAYOUT_HEAD_MAJOR, 4096, 1) == 7\n"
        "n = 0\n"
        "for n_q, ctx, splits, waves, side in ((32, 4096, 0, 0, 'measure'), (32, 5003, 7, 4, 0), (32, 1000, 3, 1, 0), (32, 3001, 5, 2, 0x55555555),\n"
        "                                      (64, 2049, 4, 8, 0xaaaaaaaa), (16, 700, 2, 4, 0), (8, 6000, 16, 4, 'measure')):\n"
        "    case = synth.make_case(29 + n, ctx=ctx, n_q=n_q, n_kv=8)\n"
        "    ref = run_oracle(oracle, case)\n"
        "    kw = dict(force_path=B.PATH_SPLIT_FUSED, num_splits=splits, waves_per_group=waves) if splits else {}\n"
        "    got16, got32, plan = run_hip(case, dev, kv_layout=B.KV_LAYOUT_HEAD_MAJOR, want_plan=True, workspace_side=side, **kw)\n"
        "    assert plan.num_splits > 1\n"
        "    assert_parity(got16, ref, 'staggered %%d/%%d/%%d/%%d' %% (n_q, ctx, splits, waves)); assert_tap_parity(got32, ref, 'tap'); n += 1\n"
        "print('ok', n)\n" % (root, os.path.join(root, "tests")))
    res = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, cwd=root,
                         env=dict(os.environ, LLMI_HIP_STAGGER_MASK="7"), timeout=280)
    assert res.returncode == 0 and "ok 7" in res.stdout, res.stdout[-3000:]


def test_qwen3_32b_head_layout_at_128k(oracle, dev):
    """64 Q / 8 KV heads at ctx 131072 (512 MiB of K and V, seed 5) at full size against the oracle:
    the dispatcher's plan (fused combine, one workgroup per CU, 8 waves), the fused combine at the
    maximum split count, and the two-launch path with the separate combine kernel at 256 splits."""
    case = synth.make_case(5, n_q=64, n_kv=8, ctx=131072)
    ref = run_oracle(oracle, case)
    for kw in (dict(), dict(force_path=B.PATH_SPLIT_FUSED, num_splits=256), dict(force_path=B.PATH_SPLIT, num_splits=256)):
        got16, got32, plan = run_hip(case, dev, kv_layout=B.KV_LAYOUT_HEAD_MAJOR, want_plan=True, **kw)
        what = "ctx=131072 path=%d splits=%d waves=%d" % (plan.path, plan.num_splits, plan.waves_per_group)
        assert_parity(got16, ref, "bf16 out " + what)
        assert_tap_parity(got32, ref, what)
        if not kw:
            assert plan.path == B.PATH_SPLIT_FUSED and plan.num_splits == 32 and plan.waves_per_group == 8
        else:
            assert plan.num_splits == 256


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(n):
        kv_mul = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 12, 16]))
        n_kv = int(rng.choice([1, 2, 3, 4, 8]))
        ctx = int(rng.choice([rng.integers(1, 64), rng.integers(64, 400), rng.integers(400, 3000)]))
        path = int(rng.choice([B.PATH_AUTO, B.PATH_SINGLE_PASS, B.PATH_SPLIT, B.PATH_SPLIT_FUSED]))
        splits = 0 if path in (B.PATH_AUTO, B.PATH_SINGLE_PASS) else int(rng.choice([0, 2, 3, 5, 11, 16, 37, 64, 256]))
        max_waves = 64 // (1 << (kv_mul - 1).bit_length())
        waves = int(rng.choice([w for w in (0, 1, 2, 4, 8) if w <= max_waves]))
        layers = int(rng.integers(1, 4))
        cases.append((i, kv_mul, n_kv, ctx, int(rng.integers(0, 40)), layers, int(rng.integers(0, layers)),
                      int(rng.choice([B.KV_LAYOUT_POS_MAJOR, B.KV_LAYOUT_HEAD_MAJOR])), path, splits, waves))
    return cases


@pytest.mark.parametrize("i,kv_mul,n_kv,ctx,slack,layers,layer_id,layout,path,splits,waves", _random_cases(48, 20240607))
def test_random_shapes_against_oracle(oracle, dev, i, kv_mul, n_kv, ctx, slack, layers, layer_id, layout, path, splits, waves):
    """48 seeded draws over group size (incl. non powers of two), KV head count, length, padding behind the last
    position, layer, layout, path, split count and wave count: combinations no hand-written case names."""
    case = synth.make_case(1000 + i, n_q=kv_mul * n_kv, n_kv=n_kv, ctx=ctx, max_seq_len=ctx + slack, layers=layers, layer_id=layer_id)
    _check(oracle, dev, case, kv_layout=layout, force_path=path, num_splits=splits, waves_per_group=waves)


def _flip_sides(word):
    """The measured sides with 1 and 2 exchanged in every region: the layout that puts everything in far memory."""
    word &= 0xFFFFFFFF
    out = 0
    for i in range(16):
        out |= {1: 2, 2: 1}.get((word >> (2 * i)) & 3, 0) << (2 * i)
    return out - (1 << 32) if out >> 31 else out


@pytest.mark.parametrize("n_q,ctx,splits,offset", [
    (32, 4096, 0, 0), (32, 1024, 0, 4096), (32, 4097, 32, 8192 + 256), (32, 777, 7, 16), (64, 9000, 0, 0), (16, 3000, 0, 12288),
    (8, 2000, 16, 0), (40, 5000, 0, 0), (32, 32768, 0, (1 << 20) + 512), (32, 4096, 256, 0),
])
def test_workspace_laid_out_by_package_side(oracle, dev, n_q, ctx, splits, offset):
    """llmi_hip_mha_workspace_side + workspace_side: two homes per row of the fused combine's workspace, each workgroup
    using the one near its XCD. The result is the plain layout's bit for bit, whichever sides are claimed -- the
    measured ones, their opposite (everything far), or a made-up word -- and the oracle's; the plan says the layout is in use."""
    case = synth.make_case(40 + ctx, n_q=n_q, n_kv=8, ctx=ctx)
    ref = run_oracle(oracle, case)
    kw = dict(kv_layout=B.KV_LAYOUT_HEAD_MAJOR, force_path=B.PATH_SPLIT_FUSED, num_splits=splits, workspace_offset=offset)
    plain16, plain32 = run_hip(case, dev, **kw)
    assert_parity(plain16, ref, "plain layout")
    ws = torch.empty(ops.workspace_bytes(n_q, 128, ctx + 1) // 4 + offset // 4, dtype=torch.float32, device=dev)[offset // 4:]
    measured = ops.workspace_side(ws)  # (0 if the timing probe made no statement on this box: then only the claims run)
    sides = ([measured, _flip_sides(measured)] if measured else []) + [0x66666666, 0x11111111 | (2 << 2), 0x55555555, -1431655766]
    for side in sides:
        got16, got32, plan = run_hip(case, dev, want_plan=True, workspace_side=side, **kw)
        assert plan.workspace_side == 1, "side word %x" % (side & 0xFFFFFFFF)
        assert np.array_equal(got16, plain16) and np.array_equal(got32, plain32), "side word %x" % (side & 0xFFFFFFFF)


def test_workspace_side_falls_back_to_the_plain_layout(oracle, dev):
    """Where the layout by side does not apply -- unknown sides, a workspace without room for two homes per row, a KV
    head count that is no multiple of eight, the separate combine kernel, a single pass, a wave count other than the
    dispatcher's own -- the call runs as before."""
    case = synth.make_case(77, n_q=32, n_kv=8, ctx=4096)
    ref = run_oracle(oracle, case)
    small = 32 * 32 * 528 + 16  # exactly the plain layout's need at 32 splits
    for kw in (dict(workspace_side=0), dict(workspace_side=1, workspace_bytes=small, num_splits=32),
               dict(workspace_side=1, force_path=B.PATH_SPLIT, num_splits=32), dict(workspace_side=1, force_path=B.PATH_SINGLE_PASS),
               dict(workspace_side=1, waves_per_group=2), dict(workspace_side=1, waves_per_group=8)):
        got16, _, plan = run_hip(case, dev, want_plan=True, kv_layout=B.KV_LAYOUT_HEAD_MAJOR, **kw)
        assert plan.workspace_side == 0
        assert_parity(got16, ref, str(kw))
    case = synth.make_case(78, n_q=12, n_kv=4, ctx=3000)
    got16, _, plan = run_hip(case, dev, want_plan=True, workspace_side=1)
    assert plan.workspace_side == 0
    assert_parity(got16, run_oracle(oracle, case), "4 KV heads")


def test_workspace_side_measurements_never_contradict(dev):
    """Twenty measurements of one workspace: every one that makes a statement about a region makes the same one, and the
    library's own tally has no contradiction (two probe runs naming opposite sides). How often the probe abstains is
    reported by the tally, not asserted: an abstention keeps the plain layout and costs nothing but time."""
    ws = torch.empty(ops.workspace_bytes(32, 128, 32768) // 4, dtype=torch.float32, device=dev)
    stats0 = (ctypes.c_uint64 * 3)()
    B.lib().llmi_hip_workspace_side_stats(stats0)
    words = [ops.workspace_side(ws) & 0xFFFFFFFF for _ in range(20)]
    stats = (ctypes.c_uint64 * 3)()
    B.lib().llmi_hip_workspace_side_stats(stats)
    for region in range(16):
        named = {(w >> (2 * region)) & 3 for w in words} - {0}
        assert len(named) <= 1, "region %d: %s" % (region, sorted(named))
    assert stats[2] == stats0[2], "contradicting probe runs"
    assert stats[0] + stats[1] > stats0[0] + stats0[1]
    print("workspace side: %d agreed, %d abstained of %d region measurements"
          % (stats[0] - stats0[0], stats[1] - stats0[1], stats[0] + stats[1] - stats0[0] - stats0[1]))


def test_workspace_side_argument_checks(dev):
    ws = torch.empty(1 << 20, dtype=torch.float32, device=dev)
    side = ctypes.c_int32(-1)
    f = B.lib().llmi_hip_mha_workspace_side
    st = torch.cuda.current_stream().cuda_stream
    assert f(None, 1 << 22, st, ctypes.byref(side)) == B.STATUS["NULL_POINTER"]
    assert f(ws.data_ptr(), 1 << 22, st, None) == B.STATUS["NULL_POINTER"]
    assert f(ws.data_ptr() + 4, 1 << 22, st, ctypes.byref(side)) == B.STATUS["ALIGNMENT"]
    assert f(ws.data_ptr(), 40 << 10, st, ctypes.byref(side)) == B.STATUS["WORKSPACE"]
    g = torch.cuda.CUDAGraph()
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        with torch.cuda.graph(g, stream=s2):
            assert f(ws.data_ptr(), 1 << 22, s2.cuda_stream, ctypes.byref(side)) == B.STATUS["INVALID_ARG"]  # not under capture
            torch.zeros(4, device=dev).add_(1)


@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("n_q,ctx,splits", [(32, 4096, 0), (32, 5000, 32), (64, 9000, 0), (32, 20000, 100), (16, 700, 5)])
def test_splits_that_used_the_other_home_are_still_found(oracle, dev, mode, n_q, ctx, splits):
    """llmi_hip_set_test_far_home: every split but the merging one (mode 1), or every second split (mode 2), keeps its
    partial results and record in the home of the OTHER side of the package, as if the workgroups of a KV head had not
    shared an XCD. The merging workgroup finds nothing (or half) in the home it polls, falls back to both homes after 16
    rounds and reads every split's rows from where its record was: the bits of the undisturbed call, no give-up counted,
    also on the next call and with the opposite sides claimed."""
    case = synth.make_case(60 + ctx, n_q=n_q, n_kv=8, ctx=ctx)
    kw = dict(kv_layout=B.KV_LAYOUT_HEAD_MAJOR, force_path=B.PATH_SPLIT_FUSED, num_splits=splits)
    want16, want32, plan = run_hip(case, dev, want_plan=True, workspace_side="measure", **kw)
    assert plan.workspace_side == 1
    assert_parity(want16, run_oracle(oracle, case), "undisturbed")
    timeouts = ctypes.c_uint64()
    assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(timeouts)) == 0
    before = timeouts.value
    assert B.lib().llmi_hip_set_test_far_home(mode) == 0
    try:
        for side in ("measure", 0x55555555, -1431655766):
            got16, got32 = run_hip(case, dev, workspace_side=side, **kw)
            assert np.array_equal(got16, want16) and np.array_equal(got32, want32), "mode %d sides %s" % (mode, side)
    finally:
        assert B.lib().llmi_hip_set_test_far_home(0) == mode
    again16, again32 = run_hip(case, dev, workspace_side="measure", **kw)
    assert np.array_equal(again16, want16) and np.array_equal(again32, want32)
    assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(timeouts)) == 0 and timeouts.value == before
