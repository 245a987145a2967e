"""The C ABI without a GPU: the library loads, exports every symbol include/llmi_hip.h declares, its
structs have the layout the binding assumes, and validation / dispatch planning (which make no HIP call)
return the documented status codes."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

from llminfer_amd import _binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("llmi_hip.h", "llmi_hip_probes.h", "llmi_hip_testing.h")]
DIAG_HEADER = os.path.join(ROOT, "include", "llmi_hip_diag.h")


def declared_functions(headers=HEADERS):
    text = "".join(open(h).read() for h in headers)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(llmi_[a-z0-9_]+)\s*\(", text)
    # typedef'd function-pointer types are not exported symbols
    return sorted(set(n for n in names if not n.endswith("_fn")))


def test_every_declared_symbol_is_exported_and_bound():
    lib = B.lib()
    names = declared_functions()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), "libllmi_hip.so does not export " + name
        assert name in B.SYMBOLS, "the ctypes binding does not declare " + name
    assert set(B.SYMBOLS) == set(names)
    header = open(HEADERS[0]).read()
    declared = int(re.search(r"#define\s+LLMI_HIP_ABI_VERSION\s+(\d+)", header).group(1))
    assert declared == 3 and lib.llmi_hip_abi_version() == declared
    # every header of include/ is covered by this test or the next one
    assert sorted(os.listdir(os.path.join(ROOT, "include"))) == sorted(os.path.basename(h) for h in HEADERS + [DIAG_HEADER])


def test_diag_library_exports_its_header():
    lib = B.diag_lib()
    names = declared_functions([DIAG_HEADER])
    assert names == sorted(B.DIAG_SYMBOLS)
    for name in names:
        assert hasattr(lib, name), "libllmi_diag.so does not export " + name
    # ... and the product library carries none of it
    for name in names + ["llmi_hip_probe_handover", "llmi_hip_probe_placement"]:
        assert not hasattr(B.lib(), name)


def test_struct_layout_matches_the_c_compiler(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(r'''
#include <stdio.h>
#include <stddef.h>
#include "llmi_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu\n", sizeof(llmi_mha_args), offsetof(llmi_mha_args, layer_id),
           offsetof(llmi_mha_args, waves_per_group), offsetof(llmi_mha_args, stream), sizeof(llmi_mha_plan));
    printf("%zu %zu %zu %zu %zu\n", offsetof(llmi_mha_args, workspace_side), sizeof(llmi_mha_append_args),
           offsetof(llmi_mha_append_args, eps), sizeof(llmi_attn_oproj_args), offsetof(llmi_attn_oproj_args, one_launch));
    printf("%zu %zu %zu %zu\n", sizeof(llmi_qk_norm_rope_args), offsetof(llmi_qk_norm_rope_args, eps),
           offsetof(llmi_qk_norm_rope_args, stream), sizeof(llmi_pool_stats));
    return 0;
}
''')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout.split()
    got = [int(x) for x in out]
    want = [ctypes.sizeof(B.MhaArgs), B.MhaArgs.layer_id.offset, B.MhaArgs.waves_per_group.offset,
            B.MhaArgs.stream.offset, ctypes.sizeof(B.MhaPlan),
            B.MhaArgs.workspace_side.offset, ctypes.sizeof(B.MhaAppendArgs), B.MhaAppendArgs.eps.offset,
            ctypes.sizeof(B.AttnOprojArgs), B.AttnOprojArgs.one_launch.offset, ctypes.sizeof(B.QkNormRopeArgs),
            B.QkNormRopeArgs.eps.offset, B.QkNormRopeArgs.stream.offset, ctypes.sizeof(B.PoolStats)]
    assert got == want


def good_args(**over):
    a = B.MhaArgs()
    a.query = a.key_cache = a.value_cache = a.output = 0x1000
    a.workspace = 0x2000
    a.workspace_bytes = 64 << 20
    a.layer_id, a.pos, a.kv_dim, a.kv_mul, a.head_num, a.head_dim, a.max_seq_len = 0, 4095, 1024, 4, 32, 128, 4096
    for k, v in over.items():
        setattr(a, k, v)
    return a


def plan(a):
    p = B.MhaPlan()
    rc = B.lib().llmi_hip_mha_plan(ctypes.byref(a), ctypes.byref(p))
    return rc, p


@pytest.mark.parametrize("over,status", [
    (dict(query=0), "NULL_POINTER"), (dict(output=0), "NULL_POINTER"),
    (dict(head_dim=64), "HEAD_DIM"),                      # mha_kernel.cu:478-479
    (dict(kv_dim=1000), "KV_DIM"), (dict(kv_dim=0), "KV_DIM"),
    (dict(head_num=31), "HEAD_GROUP"), (dict(kv_mul=0), "HEAD_GROUP"),
    (dict(kv_mul=32, head_num=256), "HEAD_GROUP"),
    (dict(pos=-1), "POS_RANGE"), (dict(pos=4096), "POS_RANGE"),  # mha_kernel.cu:473-474
    (dict(query=0x1008), "ALIGNMENT"), (dict(key_cache=0x1002), "ALIGNMENT"),  # mha_kernel.cu:495-498
    (dict(kv_layout=2), "LAYOUT"), (dict(force_path=4), "INVALID_ARG"), (dict(num_splits=257), "INVALID_ARG"),
    (dict(waves_per_group=3), "INVALID_ARG"), (dict(layer_id=-1), "INVALID_ARG"), (dict(max_seq_len=0), "INVALID_ARG"),
    (dict(workspace=0), "WORKSPACE"), (dict(workspace_bytes=1000), "WORKSPACE"),
    (dict(force_path=B.PATH_SPLIT, num_splits=64, workspace_bytes=32 * 130 * 4 * 63), "WORKSPACE"),
])
def test_validation_status_codes(over, status):
    rc, _ = plan(good_args(**over))
    assert rc == B.STATUS[status], B.lib().llmi_hip_strerror(rc)
    # the launcher validates the same way and returns before touching HIP
    assert B.lib().llmi_hip_mha_decode(ctypes.byref(good_args(**over))) == B.STATUS[status]


def test_null_arguments():
    p = B.MhaPlan()
    assert B.lib().llmi_hip_mha_plan(None, ctypes.byref(p)) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_mha_plan(ctypes.byref(good_args()), None) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_mha_decode(None) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_qk_norm_rope_append(None) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_sincos_table(None, None, 128, 16, None) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_kv_restride(None, None, 1, 16, 1024, 128, 1, None) == B.STATUS["NULL_POINTER"]
    assert B.lib().llmi_hip_memcpy(None, None, 4, 0, None, 0) == B.STATUS["NULL_POINTER"]


def test_plan_short_context_is_single_pass():
    for pos in (0, 15, 16, 127, 159, 175):  # up to 176 positions: one workgroup per KV head
        rc, p = plan(good_args(pos=pos, workspace=0, workspace_bytes=0))  # no workspace needed
        assert rc == 0 and p.path == B.PATH_SINGLE_PASS and p.num_splits == 1 and p.workspace_needed == 0
        assert p.rows_per_split >= pos + 1 and p.rows_per_split % 16 == 0


@pytest.mark.parametrize("ctx", [177, 209, 1024, 4096, 8192, 32768, 131072])
def test_plan_long_context_splits_without_empty_splits(ctx):
    rc, p = plan(good_args(pos=ctx - 1, max_seq_len=ctx))
    assert rc == 0 and p.path == B.PATH_SPLIT_FUSED and 2 <= p.num_splits <= 256
    assert p.rows_per_split % 16 == 0
    tiles = (ctx + 15) // 16
    assert p.num_splits <= tiles and p.rows_per_split == -(-tiles // p.num_splits) * 16  # no split without a tile
    assert p.workspace_needed <= B.lib().llmi_hip_mha_workspace_bytes(32, 128, ctx)
    assert p.group_pad == 4 and p.waves_per_group in (1, 2, 4, 8)


def test_plan_split_count_by_length():
    """32 query / 8 KV heads: 8 splits while 16 would leave some without a tile, 16 until they would hold more than four
    tiles each (1024 positions), then one workgroup per CU, in both layouts."""
    for layout in (0, 1):
        for ctx, splits in ((177, 8), (240, 8), (241, 16), (700, 16), (1024, 16), (1025, 32), (1041, 32), (1500, 32), (3000, 32), (4096, 32), (32768, 32)):
            rc, p = plan(good_args(pos=ctx - 1, max_seq_len=32768, kv_layout=layout))
            assert rc == 0 and p.path == B.PATH_SPLIT_FUSED and p.num_splits == splits, (layout, ctx, p.num_splits)


def test_plan_groups_of_eight_query_heads():
    """64 query / 8 KV heads: 8 waves per workgroup, a single pass up to 240 positions (15 tiles), then 16 splits
    until they would hold more than four tiles each (1024 positions), then one workgroup per CU (32 splits)."""
    eight = dict(kv_mul=8, head_num=64, max_seq_len=32768)
    for pos in (0, 127, 208, 239):
        rc, p = plan(good_args(pos=pos, **eight))
        assert rc == 0 and p.path == B.PATH_SINGLE_PASS and p.num_splits == 1 and p.group_pad == 8
    for ctx, splits in ((241, 16), (256, 16), (1024, 16), (1025, 32), (1041, 32), (4096, 32), (8192, 32), (32768, 32)):
        rc, p = plan(good_args(pos=ctx - 1, **eight))
        assert rc == 0 and p.path == B.PATH_SPLIT_FUSED and p.waves_per_group == 8
        assert p.num_splits == splits and p.rows_per_split == -(-((ctx + 15) // 16) // splits) * 16


def test_plan_with_a_measured_workspace_side():
    """workspace_side set: the fused combine's arrays move to the next 16 KiB boundary and keep two homes per row, if
    the shape qualifies (a multiple of eight KV heads, at most 128 heads, groups of at most 8 query heads with the
    wave count the dispatcher picks itself: the kernel is built for the layout with those) and the workspace has the
    room; otherwise the plain layout, without an error."""
    rc, p = plan(good_args(workspace_side=1, workspace=0x2000))
    rows = 32 * p.num_splits
    assert rc == 0 and p.path == B.PATH_SPLIT_FUSED and p.workspace_side == 1
    assert p.workspace_needed == (0x4000 - 0x2000) + 2 * -(-rows // 16) * 8192 + 2 * -(-rows // 512) * 8192 + 16
    rc, p0 = plan(good_args(workspace_side=0, workspace=0x2000))
    assert rc == 0 and p0.workspace_side == 0 and p0.num_splits == p.num_splits and p0.workspace_needed == rows * 528 + 16
    assert B.lib().llmi_hip_mha_workspace_bytes(32, 128, 4096) >= p.workspace_needed + 8192 + 32 * 4
    for over in (dict(workspace_bytes=p.workspace_needed - 1),                 # no room for two homes
                 dict(kv_mul=8, head_num=32, kv_dim=512),                       # 4 KV heads
                 dict(waves_per_group=2), dict(waves_per_group=8),              # not the dispatcher's own wave count
                 dict(kv_mul=16, head_num=128, kv_dim=1024),                    # groups of 16 query heads
                 dict(force_path=B.PATH_SPLIT, num_splits=8), dict(pos=100)):   # separate combine kernel, single pass
        rc, q = plan(good_args(workspace_side=1, workspace=0x2000, **over))
        assert rc == 0 and q.workspace_side == 0, over
    rc, p = plan(good_args(workspace_side=-1431655766, workspace=0x4000))  # (0xAAAAAAAA as int32: any word is taken)
    assert rc == 0 and p.workspace_side == 1 and p.workspace_needed == 2 * -(-rows // 16) * 8192 + 2 * -(-rows // 512) * 8192 + 16
    rc, p = plan(good_args(workspace_side=1, workspace=0x2000, waves_per_group=4))  # the dispatcher's own count, spelled out
    assert rc == 0 and p.workspace_side == 1
    rc, p = plan(good_args(workspace_side=1, workspace=0x2000, kv_mul=8, head_num=64, kv_dim=1024, workspace_bytes=8 << 20))
    assert rc == 0 and p.workspace_side == 1 and p.waves_per_group == 8


def test_plan_honours_requests_and_clamps_to_the_workspace():
    rc, p = plan(good_args(force_path=B.PATH_SPLIT, num_splits=16))
    assert rc == 0 and p.path == B.PATH_SPLIT and p.num_splits == 16 and p.rows_per_split == 256
    rc, p = plan(good_args(force_path=B.PATH_SPLIT, num_splits=200))  # 256 tiles: 56 splits of 2, 144 of 1
    assert rc == 0 and p.num_splits == 200 and p.rows_per_split == 32
    rc, p = plan(good_args(force_path=B.PATH_SINGLE_PASS))
    assert rc == 0 and p.path == B.PATH_SINGLE_PASS and p.num_splits == 1
    # a reference-sized workspace [head_num, 4*max_seq_len] fp32 (qwen3_fused.cpp:502) limits the auto split count
    small = 32 * 4 * 512 * 4
    rc, p = plan(good_args(pos=511, max_seq_len=512, workspace_bytes=small))
    assert rc == 0 and p.workspace_needed <= small and p.num_splits >= 2
    # kv_mul 3 pads to 4, kv_mul 16 limits the waves per workgroup
    rc, p = plan(good_args(kv_mul=3, head_num=24))
    assert rc == 0 and p.group_pad == 4
    rc, p = plan(good_args(kv_mul=16, head_num=128))
    assert rc == 0 and p.group_pad == 16 and p.waves_per_group <= 4
    rc, _ = plan(good_args(kv_mul=16, head_num=128, waves_per_group=8))
    assert rc == B.STATUS["INVALID_ARG"]


def test_plan_with_a_device_position():
    """pos_device: pos is the largest position the launch serves; the separate combine kernel cannot follow
    a position it does not read, and the pointer must be int32-aligned."""
    rc, p = plan(good_args(pos_device=0x1000))
    assert rc == 0 and p.path == B.PATH_SPLIT_FUSED
    rc, _ = plan(good_args(pos_device=0x1000, force_path=B.PATH_SPLIT, num_splits=8))
    assert rc == B.STATUS["INVALID_ARG"]
    rc, _ = plan(good_args(pos_device=0x1002))
    assert rc == B.STATUS["ALIGNMENT"]


def test_workspace_bytes():
    f = B.lib().llmi_hip_mha_workspace_bytes
    assert f(0, 128, 100) == 0 and f(32, 128, 0) == 0
    assert f(32, 128, 4096) >= 32 * 256 * 130 * 4
    assert f(32, 128, 1 << 20) == f(32, 128, 4096)  # the split count is capped
    assert f(32, 128, 64) < f(32, 128, 4096)


def test_strerror_covers_every_status():
    msgs = {B.lib().llmi_hip_strerror(code).decode() for code in B.STATUS.values()}
    assert len(msgs) == len(B.STATUS) and "unknown status" not in msgs
    assert B.lib().llmi_hip_strerror(-99).decode() == "unknown status"


def test_qk_norm_rope_validation():
    a = B.QkNormRopeArgs()
    for f in ("query", "key_new", "key_cache", "norm_weight", "sin_cache", "cos_cache"):
        setattr(a, f, 0x1000)
    a.layer_id, a.pos, a.kv_dim, a.head_num, a.head_dim, a.max_seq_len, a.eps = 0, 5, 1024, 32, 64, 16, 1e-6
    call = B.lib().llmi_hip_qk_norm_rope_append
    assert call(ctypes.byref(a)) == B.STATUS["HEAD_DIM"]
    a.head_dim = 128
    a.pos = 16
    assert call(ctypes.byref(a)) == B.STATUS["POS_RANGE"]
    a.pos = 5
    a.value_new = 0x1000  # V row given but no V cache to put it in
    assert call(ctypes.byref(a)) == B.STATUS["NULL_POINTER"]
    a.value_cache = 0x1000
    a.kv_layout = 7
    assert call(ctypes.byref(a)) == B.STATUS["LAYOUT"]
    a.kv_layout = 0
    a.query_src = 0x1001
    assert call(ctypes.byref(a)) == B.STATUS["ALIGNMENT"]


def test_missing_library_fails_loudly(tmp_path):
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from llminfer_amd import _binding as B\n"
            "B.LIB_PATH = %r\n"
            "try:\n    B.lib()\nexcept RuntimeError as e:\n    print('RAISED', e)\n" % (ROOT, str(tmp_path / "nope.so")))
    out = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert "RAISED" in out and "no fallback" in out


def test_gemv_argument_checks():
    """Validation happens before any HIP call (k % 8, alignment: matmul_kernel.cu:123-128)."""
    L = B.lib()
    a = B.GemvArgs()
    a.input, a.weight, a.output, a.n, a.k, a.mode = 0x1000, 0x2000, 0x3000, 16, 64, B.GEMV_OUT_BF16
    for field, value, status in (("input", 0, "NULL_POINTER"), ("weight", 0, "NULL_POINTER"), ("output", 0, "NULL_POINTER"),
                                 ("k", 60, "INVALID_ARG"), ("n", 0, "INVALID_ARG"), ("mode", 7, "INVALID_ARG"),
                                 ("weight", 0x2008, "ALIGNMENT"), ("input", 0x1002, "ALIGNMENT")):
        b = B.GemvArgs.from_buffer_copy(a)
        setattr(b, field, value)
        assert L.llmi_hip_gemv(ctypes.byref(b)) == B.STATUS[status], field
    assert L.llmi_hip_gemv(None) == B.STATUS["NULL_POINTER"]
    q = B.QkvGemvArgs()
    q.input, q.weight, q.query, q.key, q.value, q.dim, q.kv_dim, q.k = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000, 256, 128, 64
    for field, value, status in (("key", 0, "NULL_POINTER"), ("k", 4, "INVALID_ARG"), ("kv_dim", 0, "INVALID_ARG"),
                                 ("value", 0x5004, "ALIGNMENT")):
        b = B.QkvGemvArgs.from_buffer_copy(q)
        setattr(b, field, value)
        assert L.llmi_hip_qkv_gemv(ctypes.byref(b)) == B.STATUS[status], field


def test_poll_limit_round_trip():
    """The bound on the fused combine's wait: default 2^22 polls, negative values clamp to zero,
    the setter returns what was there before (no GPU involved)."""
    lib = B.lib()
    assert lib.llmi_hip_set_poll_limit(7) == 1 << 22
    assert lib.llmi_hip_set_poll_limit(-5) == 7
    assert lib.llmi_hip_set_poll_limit(1 << 22) == 0


def test_plan_invariants_over_random_arguments():
    """Whatever the shape, length, workspace and overrides: a plan that comes back LLMI_OK covers every position
    exactly once, leaves no split without a tile, fits the workspace it was given and names a kernel that exists."""
    hyp = pytest.importorskip("hypothesis")
    st = hyp.strategies

    @hyp.settings(max_examples=600, deadline=None, derandomize=True)
    @hyp.given(kv_mul=st.integers(1, 16), n_kv=st.sampled_from([1, 2, 4, 8, 16]), ctx=st.integers(1, 140000),
               slack=st.integers(0, 64), force_path=st.integers(0, 3), num_splits=st.sampled_from([0, 0, 0, 1, 2, 3, 7, 32, 200, 256]),
               waves=st.sampled_from([0, 0, 1, 2, 4, 8]), ws_kib=st.sampled_from([0, 1, 64, 4096, 1 << 17]),
               side=st.sampled_from([0, 0, 1, 2, 0x66, -1]))
    def check(kv_mul, n_kv, ctx, slack, force_path, num_splits, waves, ws_kib, side):
        a = good_args(pos=ctx - 1, max_seq_len=ctx + slack, kv_mul=kv_mul, kv_dim=128 * n_kv, head_num=kv_mul * n_kv,
                      force_path=force_path, num_splits=num_splits, waves_per_group=waves,
                      workspace=0x2000 if ws_kib else 0, workspace_bytes=ws_kib << 10, workspace_side=side)
        rc, p = plan(a)
        if rc != 0:
            assert rc in (B.STATUS["WORKSPACE"], B.STATUS["INVALID_ARG"])
            return
        tiles = (ctx + 15) // 16
        assert 1 <= p.num_splits <= min(256, tiles)
        assert p.rows_per_split % 16 == 0 and p.rows_per_split == -(-tiles // p.num_splits) * 16
        assert (p.num_splits == 1) == (p.path == B.PATH_SINGLE_PASS)
        assert p.workspace_needed <= (ws_kib << 10) and (p.num_splits == 1) == (p.workspace_needed == 0)
        assert p.workspace_side in (0, 1) and (p.workspace_side == 0 or (side != 0 and n_kv % 8 == 0 and p.path == B.PATH_SPLIT_FUSED
                                                                 and p.waves_per_group == (8 if p.group_pad == 8 else 4)))
        assert p.group_pad in (1, 2, 4, 8, 16) and kv_mul <= p.group_pad < 2 * kv_mul
        assert p.waves_per_group in (1, 2, 4, 8) and p.group_pad * p.waves_per_group <= 64
        if waves:
            assert p.waves_per_group == waves
        if num_splits and force_path != B.PATH_SINGLE_PASS:
            assert p.num_splits == min(num_splits, tiles)
        if force_path == B.PATH_SINGLE_PASS:
            assert p.num_splits == 1
        if force_path in (B.PATH_SPLIT, B.PATH_SPLIT_FUSED) and p.num_splits > 1:
            assert p.path == force_path

    check()


def test_build_rejects_kernels_with_a_private_segment():
    """The build reads the compiler's resource-usage remarks and refuses a kernel that was given scratch memory."""
    from llminfer_amd import build
    remarks = "\n".join([
        "a.hip:1:1: remark: Function Name: kern_a [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:9:1: remark: Function Name: kern_b [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:9:1: remark:     VGPRs: 14 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:9:1: remark:     ScratchSize [bytes/lane]: 48 [-Rpass-analysis=kernel-resource-usage]"])
    assert build.kernels_using_scratch(remarks) == ["kern_b"]
    assert build.kernels_using_scratch("") == []


@pytest.mark.parametrize("head_dim", [64, 128, 256, 4096, 2**31 - 1])
def test_workspace_bytes_for_any_head_dim(head_dim):
    """The size query never divides by a block count of zero (a row wider than the 8 KiB blocks of the layout by side
    has none): any head_dim gives a size that holds the plain layout."""
    n = B.lib().llmi_hip_mha_workspace_bytes(32, head_dim, 4096)
    assert n >= 32 * 256 * (head_dim * 4 + 16) + 16
    if head_dim == 128:
        assert n >= 2 * (32 * 256 // 16) * 8192  # two homes per row


def test_environment_overrides_of_the_dispatch():
    """LLMI_HIP_SINGLE_PASS_MAX and LLMI_HIP_NUM_SPLITS move the threshold and the split count where the caller
    left both to the dispatcher, and nothing else (read once per process: a child process per setting)."""
    code = (
        "import ctypes, sys; sys.path.insert(0, %r)\n"
        "from tests.test_c_abi import good_args, plan\n"
        "out = []\n"
        "for pos, over in ((99, {}), (299, {}), (4095, {}), (4095, dict(num_splits=8)), (299, dict(force_path=1)), (4095, dict(workspace_bytes=5 * 32 * 528 + 16))):\n"
        "    rc, p = plan(good_args(pos=pos, **over)); out.append('%%d:%%d:%%d' %% (rc, p.path, p.num_splits))\n"
        "print(' '.join(out))\n" % ROOT)

    def run(**env):
        e = dict(os.environ, **env)
        return subprocess.run([sys.executable, "-c", code], check=True, stdout=subprocess.PIPE, text=True, env=e, cwd=ROOT).stdout.split()

    assert run() == ["0:1:1", "0:3:16", "0:3:32", "0:3:8", "0:1:1", "0:3:5"]
    assert run(LLMI_HIP_SINGLE_PASS_MAX="400") == ["0:1:1", "0:1:1", "0:3:32", "0:3:8", "0:1:1", "0:3:5"]
    assert run(LLMI_HIP_SINGLE_PASS_MAX="50") == ["0:3:7", "0:3:16", "0:3:32", "0:3:8", "0:1:1", "0:3:5"]
    assert run(LLMI_HIP_NUM_SPLITS="12") == ["0:1:1", "0:3:12", "0:3:12", "0:3:8", "0:1:1", "0:3:5"]
    assert run(LLMI_HIP_NUM_SPLITS="junk", LLMI_HIP_SINGLE_PASS_MAX="-3") == run()


def test_stagger_rule_of_the_split_path():
    """Which lengths get the staggered walk: position-major where the splits' runs are exactly 512 KiB or 1 MiB,
    head-major from 512 KiB to below 2 MiB at (or a few tiles above) a multiple of 512 KiB; LLMI_HIP_STAGGER_MASK overrides the
    head-major mask only (read once per process: a child process per setting)."""
    m = B.lib().llmi_hip_stagger_mask
    K = 1 << 10
    # position-major: 32 splits of 8192 positions x 2 KiB rows = 512 KiB each
    assert m(B.KV_LAYOUT_POS_MAJOR, 512 * K, 0) == 3 and m(B.KV_LAYOUT_POS_MAJOR, 1024 * K, 0) == 3
    assert m(B.KV_LAYOUT_POS_MAJOR, 512 * K, 1) == 0 and m(B.KV_LAYOUT_POS_MAJOR, 2048 * K, 0) == 0
    assert m(B.KV_LAYOUT_POS_MAJOR, 384 * K, 0) == 0 and m(B.KV_LAYOUT_POS_MAJOR, 0, 0) == 0
    # head-major: 65536 positions in 32 splits = 512 KiB runs; 131072 = 1 MiB; 196608 = 1.5 MiB; 163840 = 1.25 MiB; 262144 = 2 MiB
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 512 * K, 0) == 31 and m(B.KV_LAYOUT_HEAD_MAJOR, 1024 * K, 0) == 31
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 1536 * K, 0) == 31
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 1024 * K + 7 * 4096, 1) == 31  # the position has moved on by some tokens
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 1024 * K + 8 * 4096, 1) == 0
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 1280 * K, 0) == 0 and m(B.KV_LAYOUT_HEAD_MAJOR, 768 * K, 0) == 0
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 2048 * K, 0) == 0 and m(B.KV_LAYOUT_HEAD_MAJOR, 4096 * K, 0) == 0
    assert m(B.KV_LAYOUT_HEAD_MAJOR, 256 * K, 0) == 0 and m(B.KV_LAYOUT_HEAD_MAJOR, 0, 0) == 0
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from llminfer_amd import _binding as B\n"
            "m = B.lib().llmi_hip_stagger_mask\n"
            "print(m(1, 1 << 20, 0), m(1, 256 << 10, 0), m(0, 512 << 10, 0), m(0, 2 << 20, 0))\n" % ROOT)

    def run(**env):
        e = dict(os.environ, **env)
        return subprocess.run([sys.executable, "-c", code], check=True, stdout=subprocess.PIPE, text=True, env=e, cwd=ROOT).stdout.split()

    assert run() == ["31", "0", "3", "0"]
    assert run(LLMI_HIP_STAGGER_MASK="0") == ["0", "0", "3", "0"]
    assert run(LLMI_HIP_STAGGER_MASK="7") == ["7", "7", "3", "0"]
    assert run(LLMI_HIP_STAGGER_MASK="junk") == run()


def test_side_decision_from_injected_timings():
    """The decision behind llmi_hip_mha_workspace_side as a pure function of the ping-pong probe's result words:
    clear cases, noise below the threshold, ties, pairs that lost a number or did not share an XCD, a side of the
    package without two usable pairs."""
    lib = B.lib()

    def rows(spec):
        """spec: per pair (xcd, ticks through the clear block, ticks through the set block[, ok[, partner xcd]])"""
        r = (ctypes.c_uint32 * 64)()
        for p, t in enumerate(spec):
            xcd, a, b = t[:3]
            ok = t[3] if len(t) > 3 else 1
            partner = t[4] if len(t) > 4 else xcd
            r[8 * p + 0], r[8 * p + 1], r[8 * p + 2], r[8 * p + 3], r[8 * p + 5] = xcd, a, b, ok, partner
        return r

    def decide(spec):
        return lib.llmi_hip_side_from_pingpong(rows(spec))

    # 64 hand-overs per block and run, ticks of 10 ns: 25 ns per hand-over = 160 ticks
    near, far = 3600, 4400
    assert decide([(x, near, far) for x in range(4)] + [(x, far, near) for x in range(4, 8)]) == 1
    assert decide([(x, far, near) for x in range(4)] + [(x, near, far) for x in range(4, 8)]) == 2
    assert decide([(x, near, near + 100) for x in range(4)] + [(x, near + 100, near) for x in range(4, 8)]) == 0   # below the threshold
    assert decide([(x, near, near + 160) for x in range(4)] + [(x, near + 160, near) for x in range(4, 8)]) == 1   # exactly at it
    assert decide([(x, near, near) for x in range(8)]) == 0                                                       # a tie
    assert decide([(x, near, far) for x in range(8)]) == 0                       # both sides prefer the same block
    assert decide([(x, near, far) for x in range(4)] + [(x, near, near + 10) for x in range(4, 8)]) == 0          # one side unclear
    # noise on single pairs does not flip a clear average
    assert decide([(0, far, near), (1, near, far + 900), (2, near, far), (3, near, far)] + [(x, far, near) for x in range(4, 8)]) == 1
    # pairs that lost a number or did not share an XCD do not count; two good pairs per side are enough
    assert decide([(0, near, far), (1, near, far), (2, 0, 0, 0), (3, far, near, 1, 5)] + [(4, far, near), (5, far, near), (6, 9, 9, 0), (7, 1, 9999, 1, 0)]) == 1
    assert decide([(0, near, far), (1, 0, 0, 0), (2, 0, 0, 0), (3, 0, 0, 0)] + [(x, far, near) for x in range(4, 8)]) == 0  # one pair on a side
    assert decide([(x, near, far) for x in range(4)] + [(x, 0, 0, 0) for x in range(4, 8)]) == 0                  # one side missing
    assert decide([(12, near, far)] * 8) == 0                                                                     # no such XCD
    assert lib.llmi_hip_side_from_pingpong(None) == 0

    def agree(ds):
        v = ctypes.c_int32(-1)
        arr = (ctypes.c_int32 * max(1, len(ds)))(*ds)
        return lib.llmi_hip_side_agreement(arr, len(ds), ctypes.byref(v)), v.value

    assert agree([1, 1]) == (1, 0) and agree([2, 0, 2]) == (2, 0) and agree([0, 1, 0, 1]) == (1, 0)
    assert agree([1]) == (0, 1) and agree([0, 0, 0, 0]) == (0, 1) and agree([0, 2, 0, 0]) == (0, 1) and agree([]) == (0, 1)
    assert agree([1, 2]) == (0, 2) and agree([1, 1, 2]) == (0, 2) and agree([0, 2, 1, 2]) == (0, 2)
    assert agree([7, 1, -1, 1]) == (1, 0)                                                                         # junk is no statement
