#!/usr/bin/env python3
"""Benchmark of the decode-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--ctx 1024,...,32768]

One "step" is one layer call of llmi_hip_mha_decode (through the C ABI) at
every context length of the sweep, Qwen3-4B layer shape (32 Q heads, 8 KV
heads, head_dim 128), batch 1, bf16 KV cache in the head-major layout, inputs
resident in HBM. Calls rotate over distinct slices of a KV arena much larger
than the 256 MB Infinity Cache, so every call streams from HBM. The calls are
captured into a HIP graph (no host code between kernels) and timed with HIP
events on the stream that replays it.

Prints ONE JSON line. `value` is algorithmic bytes per step / time per step.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_Q, N_KV, HEAD_DIM = 32, 8, 128
KV_DIM = N_KV * HEAD_DIM
HBM_PEAK_GBS = 8000.0
DEFAULT_CTX = [1024, 2048, 4096, 8192, 16384, 32768]
SLICES = 8  # steps (one KV slice per context each) inside one captured graph of the sweep
SLICE_SET_BYTES = 512 << 20  # a context's slices together are at least this big: twice the 256 MB Infinity Cache


def n_slices(ctx):
    """Distinct KV slices of one context length: at least SLICES, and enough that replaying one length alone
    still walks more K/V bytes than the Infinity Cache holds before a slice comes round again."""
    per_slice = 2 * ctx * KV_DIM * 2
    return min(128, max(SLICES, -(-SLICE_SET_BYTES // per_slice)))  # (128 slices at most: below 1024 positions a call is all latency)


def algorithmic_bytes(ctx, n_q=N_Q, n_kv=N_KV):
    """K and V rows once, q read once, out written once (bf16)."""
    return 2 * ctx * n_kv * HEAD_DIM * 2 + 2 * n_q * HEAD_DIM * 2


def make_arena(torch, dev, ctx_list, n_q=N_Q):
    """One K and one V slab; each (ctx, slice) pair owns a distinct region. Values: N(0,1),
    RMS-normalised per 128-wide head vector, rounded to bf16."""
    total_rows = sum(c * n_slices(c) for c in ctx_list)
    gen = torch.Generator(device=dev)
    gen.manual_seed(20260614)

    def slab():
        out = torch.empty((total_rows * N_KV, HEAD_DIM), dtype=torch.bfloat16, device=dev)
        chunk = 1 << 20
        for lo in range(0, out.shape[0], chunk):
            x = torch.randn((min(chunk, out.shape[0] - lo), HEAD_DIM), generator=gen, device=dev)
            x = x * torch.rsqrt((x * x).mean(dim=1, keepdim=True))
            out[lo:lo + chunk] = x.to(torch.bfloat16)
        return out.reshape(-1)

    k, v = slab(), slab()
    regions = {}
    row = 0
    for ctx in ctx_list:
        for s in range(n_slices(ctx)):
            regions[(ctx, s)] = row * KV_DIM  # element offset of a [N_KV][ctx][128] cache
            row += ctx
    q = torch.randn((n_q, HEAD_DIM), generator=gen, device=dev)
    q = (q * torch.rsqrt((q * q).mean(dim=1, keepdim=True))).to(torch.bfloat16).reshape(-1)
    return k, v, q, regions


KERNEL_SOURCES = ("mha_decode_kernels.h", "mha_device_helpers.h", "mha_decode.hip", "c_api.cpp")


def kernel_source_blob():
    """git's blob ids of the decode kernel's sources and of the dispatcher's (what `git rev-parse
    HEAD:llminfer_amd/csrc/<file>` prints for committed files), computed from the files themselves and joined
    by a '+': the kernel and the plan it is launched with decide the traffic."""
    import hashlib
    ids = []
    for name in KERNEL_SOURCES:
        data = open(os.path.join(ROOT, "llminfer_amd", "csrc", name), "rb").read()
        ids.append(hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest())
    return "+".join(ids)


def measured_traffic(ctx_list):
    """HBM bytes per launch of the decode kernel over the default sweep, as counted by rocprofv3
    (FETCH_SIZE + WRITE_SIZE, each scaled by a calibration copy): bench.py cannot run the profiler on
    itself, so it reports the figure of the committed counter summary -- only for the workload that
    summary was taken on, and only while the kernel's and the dispatcher's sources are the ones it was taken
    from (the summary names their git blob ids); otherwise None."""
    if ctx_list != DEFAULT_CTX:
        return None
    path = os.path.join(ROOT, "profiles", "mha_decode_kernel_qwen3-4b_ctx1k-32k_hbm_counters.md")
    traffic = blob = None
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                traffic = int(line.split(":")[1])
            if line.startswith("kernel_source_blob:"):
                blob = line.split(":")[1].strip()
    except OSError:
        return None
    return traffic if blob == kernel_source_blob() else None


def cpu_baseline(ctx_list, budget_s=12.0, n_q=N_Q):
    """The CPU oracle (a port of the reference's single-threaded CPU attention path) timed on this
    host on the same shapes: whole sweeps until about `budget_s` seconds have been spent."""
    import numpy as np
    import oracle
    from llminfer_amd import synth
    cases = []
    for ctx in ctx_list:
        c = synth.make_case(1000 + ctx, n_q=n_q, n_kv=N_KV, ctx=ctx)
        cases.append(c)
    oracle.lib()
    passes, t_total = 0, 0.0
    while t_total < budget_s and passes < 50:
        t0 = time.perf_counter()
        for c in cases:
            oracle.mha_cpu(c["q"], c["k"], c["v"], c["layer_id"], c["pos"], c["kv_dim"], c["kv_mul"],
                           c["head_num"], c["head_dim"], c["max_seq_len"])
        t_total += time.perf_counter() - t0
        passes += 1
    nbytes = sum(algorithmic_bytes(c, n_q) for c in ctx_list) * passes
    # The reference's own CPU-runnable case: 16 Q / 8 KV heads, 256 cached positions + 1, fp32.
    c1 = synth.make_case(1, n_q=16, n_kv=N_KV, ctx=257, max_seq_len=512, rms_norm=False)
    q1, k1, v1 = (np.ascontiguousarray(synth.bf16_bits_to_f32(c1[x])) for x in ("q", "k", "v"))
    t0 = time.perf_counter()
    for _ in range(200):
        oracle.mha_cpu(q1, k1, v1, c1["layer_id"], c1["pos"], c1["kv_dim"], c1["kv_mul"], c1["head_num"],
                       c1["head_dim"], c1["max_seq_len"])
    small_us = (time.perf_counter() - t0) / 200 * 1e6
    return {
        "value": round(nbytes / t_total / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "%d passes of the same ctx sweep %s through the CPU oracle (bf16 inputs widened to fp32), "
                  "%.1f s, %.0f us per layer call on average; 16 Q / 8 KV heads at 257 positions in fp32: "
                  "%.0f us per call"
                  % (passes, ctx_list, t_total, t_total / (passes * len(ctx_list)) * 1e6, small_us),
    }


GEMV_SHAPES = {  # name -> (rows, k, what): the projections around the attention, Qwen3-4B (hidden 2560)
    "qkv": (4096 + 2 * 1024, 2560, "packed QKV projection [dim + 2*kv_dim][hidden], rows dealt to q / k / v"),
    "oproj": (2560, 4096, "output projection [hidden][dim] with the residual add folded in"),
}


def run_gemv(args):
    """The bf16 GEMVs either side of the attention, each as a weight stream: 36 layers' worth of weights
    (more than the 256 MB Infinity Cache) are walked in one HIP graph, like the layer loop does."""
    import torch
    from llminfer_amd import _binding as B
    from llminfer_amd import ops
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    B.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n, k, what = GEMV_SHAPES[args.gemv]
    layers = 36
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    w = (torch.randn((layers, n, k), generator=gen, device=dev) * 0.05).to(torch.bfloat16)
    x = torch.randn(k, generator=gen, device=dev).to(torch.bfloat16)
    q = torch.zeros(4096, dtype=torch.bfloat16, device=dev)
    kk = torch.zeros(1024, dtype=torch.bfloat16, device=dev)
    v = torch.zeros(1024, dtype=torch.bfloat16, device=dev)
    res = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.Stream()

    def enqueue():
        for l in range(layers):
            if args.gemv == "qkv":
                ops.qkv_gemv(x, w[l], q, kk, v, stream=stream)
            else:
                ops.gemv(x, w[l], res, mode=B.GEMV_ADD_BF16, stream=stream)

    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        enqueue()
        stream.synchronize()
        with torch.cuda.graph(g, stream=stream):
            enqueue()

    def timed(replays):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(stream):
            e0.record(stream)
            for _ in range(replays):
                g.replay()
            e1.record(stream)
        e1.synchronize()
        return e0.elapsed_time(e1)

    timed(max(1, args.warmup // layers))
    replays = max(1, args.steps // layers)
    ms = timed(replays)
    us = ms * 1e3 / (replays * layers)
    # algorithmic bytes of one launch: the weight matrix once, the input, the output (read + written for the add)
    nbytes = n * k * 2 + k * 2 + n * 2 * (2 if args.gemv == "oproj" else 1)
    gbs = nbytes / (us * 1e-6) / 1e9
    print(json.dumps({
        "metric": "bf16 GEMV around decode attention, us per launch + HBM GB/s", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": replays * layers, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s, %d x %d bf16, batch 1, 36 distinct weight matrices walked per HIP graph replay"
                               % (what, n, k)},
        "us_per_launch": round(us, 3),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "gemv_kernel",
                     "avg_launch_us": round(us, 3), "avg_launch_bytes": nbytes},
    }))
    return 0


def stack_result(args, ctx):
    """The attention part of a 36-layer decode step at a fixed position, as one HIP graph. `args` needs
    stack, heads, layout, stack_mode, stack_follow_pos, steps, warmup. Returns the JSON object (or None)."""
    import numpy as np
    from llminfer_amd import _binding as B
    from llminfer_amd import synth
    host = ctypes.CDLL(os.path.join(ROOT, "llminfer_amd", "libllmi_host.so"))
    host.llmi_host_stack_create.restype = ctypes.c_void_p
    host.llmi_host_stack_create.argtypes = [ctypes.c_int32] * 5
    host.llmi_host_stack_ptr.restype = ctypes.c_void_p
    host.llmi_host_stack_ptr.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    host.llmi_host_stack_build_sincos.argtypes = [ctypes.c_void_p]
    host.llmi_host_stack_run.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    host.llmi_host_stack_capture.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
    host.llmi_host_stack_replay.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_float)]
    host.llmi_host_stack_destroy.argtypes = [ctypes.c_void_p]
    host.llmi_host_last_error.restype = ctypes.c_char_p
    layers, n_q, msl, pos = args.stack, args.heads, ctx + 8, ctx
    st = host.llmi_host_stack_create(layers, msl, n_q, N_KV, args.layout)
    if not st:
        print("bench.py: " + host.llmi_host_last_error().decode(), file=sys.stderr)
        return None

    def up(ptr, arr):
        arr = np.ascontiguousarray(arr)
        B.check(B.lib().llmi_hip_memcpy(ptr, arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes, 1, None, 1), "upload")

    def ok(rc):
        if rc != 0:
            raise RuntimeError(host.llmi_host_last_error().decode())

    hidden = 2560 if n_q == 32 else 5120 if n_q == 64 else 1024
    if args.stack_mode in (3, 4):
        host.llmi_host_stack_enable_projections.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        ok(host.llmi_host_stack_enable_projections(st, hidden))
    ok(host.llmi_host_stack_build_sincos(st))
    rng = np.random.RandomState(4)
    rows = rng.standard_normal((msl * N_KV, HEAD_DIM)).astype(np.float32)
    rows /= np.sqrt((rows * rows).mean(axis=1, keepdims=True))
    layer_bits = synth.f32_to_bf16_bits(rows).reshape(-1)  # one layer's worth, reused (rolled) for every layer
    for which in (0, 1):
        base = host.llmi_host_stack_ptr(st, which, 0)
        for l in range(layers):
            up(base + l * layer_bits.nbytes, np.roll(layer_bits, 128 * (l + 17 * which)))
    for l in range(layers):
        up(host.llmi_host_stack_ptr(st, 2, l), synth.f32_to_bf16_bits(rng.standard_normal(n_q * HEAD_DIM).astype(np.float32)))
        up(host.llmi_host_stack_ptr(st, 3, l), synth.f32_to_bf16_bits(rng.standard_normal(KV_DIM).astype(np.float32)))
        up(host.llmi_host_stack_ptr(st, 4, l), synth.f32_to_bf16_bits(rng.standard_normal(KV_DIM).astype(np.float32)))
        up(host.llmi_host_stack_ptr(st, 5, l),
           synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(2 * HEAD_DIM)).astype(np.float32)))
    if args.stack_mode in (3, 4):
        dim = n_q * HEAD_DIM
        for l in range(layers):
            up(host.llmi_host_stack_ptr(st, 12, l), synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32)))
        # one random matrix of each kind, rolled per layer (the values do not matter to the stream, the
        # addresses do: every layer reads its own 31 + 21 MB)
        wqkv = synth.f32_to_bf16_bits((rng.standard_normal((dim + 2 * KV_DIM) * hidden) / np.sqrt(hidden)).astype(np.float32))
        wo = synth.f32_to_bf16_bits((rng.standard_normal(hidden * dim) / np.sqrt(dim)).astype(np.float32))
        for l in range(layers):
            up(host.llmi_host_stack_ptr(st, 10, l), np.roll(wqkv, 8 * l))
            up(host.llmi_host_stack_ptr(st, 11, l), np.roll(wo, 8 * l))
        up(host.llmi_host_stack_ptr(st, 13, 0), synth.f32_to_bf16_bits(rng.standard_normal(hidden).astype(np.float32)))
    ok(host.llmi_host_stack_run(st, pos, args.stack_mode))
    if args.stack_follow_pos:
        host.llmi_host_stack_capture_following.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32]
        host.llmi_host_stack_set_pos.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        ok(host.llmi_host_stack_set_pos(st, pos))
        ok(host.llmi_host_stack_capture_following(st, msl - 1, args.stack_mode))
    else:
        ok(host.llmi_host_stack_capture(st, pos, args.stack_mode))
    ms = ctypes.c_float()
    ok(host.llmi_host_stack_replay(st, max(1, args.warmup), ctypes.byref(ms)))
    ok(host.llmi_host_stack_replay(st, args.steps, ctypes.byref(ms)))
    us_token = ms.value * 1e3 / args.steps
    per_layer = algorithmic_bytes(pos + 1, n_q) + 23552  # + QK-Norm/RoPE/append traffic per layer
    if args.stack_mode in (3, 4):  # + both weight matrices, the hidden input and the residual (read + written)
        per_layer += ((n_q * HEAD_DIM + 2 * KV_DIM) * hidden + hidden * n_q * HEAD_DIM) * 2 + 3 * hidden * 2
    gbs = layers * per_layer / (us_token * 1e-6) / 1e9
    host.llmi_host_stack_destroy(st)
    return {
        "metric": "attention stack of one decode step, us per token", "value": round(us_token, 2), "unit": "us/token",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us_token / 1e3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%d layers x (fused QK-Norm + RoPE + K/V append, GQA decode attention), %d Q / 8 KV "
                               "heads, ctx %d + 1 new token, %d per-layer caches (one random cache rolled per layer: distinct "
                               "addresses and values, 604 MB walked per token at 36 layers), one HIP graph per token, %s layout, %s"
                               % (layers, n_q, ctx, layers, "head-major" if args.layout == 1 else "position-major",
                                  "one launch per layer" if args.stack_mode == 2 else
                                  "ONE resident launch for all layers (llmi_hip_mha_decode_append_stack): the next layer's K/V tiles "
                                  "stream while this layer's results are merged, and a layer reads its query / K row / V row only after "
                                  "every head of the layer before has published its output" if args.stack_mode == 5 else
                                  "three launches per layer: packed QKV GEMV (hidden %d), attention, output projection + "
                                  "residual" % hidden if args.stack_mode == 3 else
                                  "two launches per layer: packed QKV GEMV (hidden %d), attention whose idle workgroups do the "
                                  "output projection + residual" % hidden if args.stack_mode == 4 else "two launches per layer")
                            + (", position read from device memory" if args.stack_follow_pos else "")},
        "us_per_layer": round(us_token / layers, 3),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
    }


def run_stack(args, ctx):
    res = stack_result(args, ctx)
    if res is None:
        return 1
    print(json.dumps(res))
    return 0


SWEEP_GRAPH_STEPS = 40
SETTLE_MS = 40.0
SETTLE_FIRST_MS = 600.0
MIN_GRAPH_STEPS = 64


class Sweep:
    """Decode-attention calls over rotating KV slices, captured into HIP graphs and timed with HIP events."""

    def __init__(self, ctx_list, n_q=N_Q, layout=1, plain_workspace=False):
        import torch
        from llminfer_amd import _binding as B
        from llminfer_amd import ops
        self.torch, self.B, self.ops = torch, B, ops
        self.ctx_list, self.n_q, self.layout = list(ctx_list), n_q, layout
        self.dev = torch.device("cuda:0")
        self.k, self.v, self.q, self.regions = make_arena(torch, self.dev, self.ctx_list, n_q)
        self.out = torch.empty(n_q * HEAD_DIM, dtype=torch.bfloat16, device=self.dev)
        self.ws = torch.empty(ops.workspace_bytes(n_q, HEAD_DIM, max(self.ctx_list)) // 4, dtype=torch.float32, device=self.dev)
        self.sink = torch.zeros(64, dtype=torch.int32, device=self.dev)
        self.stream = torch.cuda.Stream()
        self.settled = False  # (no figure taken on this arena yet: see us_per_call)
        self.decode = B.lib().llmi_hip_mha_decode
        # Set-up, once per workspace allocation, like an engine would do it: which 8 KiB blocks of the workspace lie
        # near which side of the package (the fused combine keeps its hand-over data in near memory then).
        self.side = 0 if plain_workspace else ops.workspace_side(self.ws)

    def call_args(self, ctx, s, **over):
        off = self.regions[(ctx, s)] * 2
        over.setdefault("workspace_side", self.side)
        return self.ops.make_mha_args(self.q, self.k.data_ptr() + off, self.v.data_ptr() + off, self.out, self.ws, layer_id=0,
                                      pos=ctx - 1, kv_dim=KV_DIM, kv_mul=self.n_q // N_KV, head_num=self.n_q, head_dim=HEAD_DIM,
                                      max_seq_len=ctx, kv_layout=self.layout, **over)

    def plan(self, ctx, **over):
        return self.ops.mha_plan(self.call_args(ctx, 0, **over))

    def enqueue(self, ctxs, first_step, steps, **over):
        """Steps first_step .. first_step+steps-1: one call per context each, on slice step % n_slices(ctx)."""
        for s in range(first_step, first_step + steps):
            for ctx in ctxs:
                a = self.call_args(ctx, s % n_slices(ctx), **over)
                a.stream = self.stream.cuda_stream
                self.B.check(self.decode(ctypes.byref(a)), "llmi_hip_mha_decode")

    def enqueue_floor(self, ctxs, first_step, steps, workgroups, waves, inflight):
        probe = self.B.lib().llmi_hip_probe_stream_read
        probe_rows = self.B.lib().llmi_hip_probe_stream_read_rows
        for s in range(first_step, first_step + steps):
            for ctx in ctxs:
                off = self.regions[(ctx, s % n_slices(ctx))] * 2
                if self.layout == 0:  # position-major: the same bytes as 256-byte pieces of 2 KiB rows, a grid row per KV head
                    self.B.check(probe_rows(self.k.data_ptr() + off, self.v.data_ptr() + off, ctx, N_KV, max(1, workgroups // N_KV),
                                            waves, inflight, self.sink.data_ptr(), self.stream.cuda_stream),
                                 "llmi_hip_probe_stream_read_rows")
                    continue
                self.B.check(probe(self.k.data_ptr() + off, self.v.data_ptr() + off, ctx * KV_DIM * 2, workgroups, waves,
                                   inflight, self.sink.data_ptr(), self.stream.cuda_stream), "llmi_hip_probe_stream_read")

    def capture(self, enqueue_fn, steps=SLICES):
        """A graph of `steps` steps (eager once first: loads the code objects before capture)."""
        torch = self.torch
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(self.stream):
            enqueue_fn(0, 1)
            self.stream.synchronize()
            with torch.cuda.graph(g, stream=self.stream):
                enqueue_fn(0, steps)
        return g

    def time_replays(self, graphs_and_counts):
        """Elapsed ms of the given replays, in order, between two events on the replaying stream."""
        torch = self.torch
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(self.stream):
            e0.record(self.stream)
            for g, n in graphs_and_counts:
                for _ in range(n):
                    g.replay()
            e1.record(self.stream)
        e1.synchronize()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1)

    def us_per_call(self, enqueue_fn, calls_per_step=1, reps=3, replays=None, steps=SLICES, stat="best"):
        """Best (or, stat="all", every one) of `reps` batches of graph replays (a graph of `steps` steps), us per call."""
        # At least MIN_GRAPH_STEPS calls per graph (the slices taken in turn, several times round): between two replays
        # of a graph the device idles for some microseconds, which a decode step pays once per token, not once per layer
        # -- with 8 calls per graph a call at 32768 positions reads 23.2 us, with 64 of them 22.6.
        steps = max(steps, MIN_GRAPH_STEPS)
        g = self.capture(enqueue_fn, steps)
        scale = max(1, steps // SLICES)
        n = max(1, (replays or 40) // scale)
        # Untimed replays first. After a pause (allocation, capture, host work) the device needs some ten milliseconds of
        # the same load before its clocks have settled (SETTLE_MS, before every figure); after the seconds of other work
        # and the allocation that precede a new arena it runs 4-5 % slow for a third of a second -- 64 Q heads at 131072
        # positions: 84.5 us per call for 340-390 ms, 80.0 from then on; 32 Q heads at 32768: 24.25, then 23.2 --, so
        # the first figure taken on an arena waits SETTLE_FIRST_MS.
        spent = self.time_replays([(g, max(1, 8 // scale))])
        target = SETTLE_MS if self.settled else SETTLE_FIRST_MS
        self.settled = True
        while spent < target:
            spent += max(self.time_replays([(g, n)]), 0.05)
        samples = [self.time_replays([(g, n)]) * 1e3 / (n * steps * calls_per_step) for _ in range(reps)]
        return samples if stat == "all" else min(samples)


# stream-only configurations tried for the floor: (workgroups, waves per workgroup, tiles in flight per wave)
FLOOR_CONFIGS = [(256, 4, 2), (256, 8, 2), (512, 4, 2), (256, 4, 4), (512, 8, 1), (1024, 4, 1), (512, 4, 4), (256, 8, 4)]


# ... and of the decode kernel's own grid (8 KV heads x 32 splits, LDS-DMA loads), with the splits' walks staggered by
# split & mask tiles: (waves, tiles in flight, mask). Workgroups that walk their runs in step feel the resonances of the
# request pattern with the memory channels; these do not, and are often the faster stream.
FLOOR_STAGGERED = [(4, 2, 7), (4, 2, 31), (8, 1, 31)]


def stream_floor(sw, ctx_list, configs=FLOOR_CONFIGS, staggered=FLOOR_STAGGERED):
    """Per context: the fastest stream-only launch (same K/V bytes read once and thrown away, same graph-replay
    timing as the decode figures) over a handful of launch shapes and walks."""
    rows = []
    probe_tiles = sw.B.lib().llmi_hip_probe_stream_tiles
    for ctx in ctx_list:
        best = None
        for wg, waves, inflight in configs:
            tiles = ctx * KV_DIM * 2 // 4096
            if wg > tiles:
                continue
            us = sw.us_per_call(lambda f, n: sw.enqueue_floor([ctx], f, n, wg, waves, inflight), reps=2, steps=n_slices(ctx))
            if best is None or us < best[0]:
                best = (us, wg, waves, inflight, 0)
        for waves, inflight, mask in staggered:
            if ctx // 16 < 32 * waves * 2:  # (fewer than two tiles per wavefront: nothing to stagger)
                continue

            def enq(first, n, waves=waves, inflight=inflight, mask=mask):
                for st in range(first, first + n):
                    off = sw.regions[(ctx, st % n_slices(ctx))] * 2
                    sw.B.check(probe_tiles(sw.k.data_ptr() + off, sw.v.data_ptr() + off, ctx, N_KV, sw.layout, 32, waves, inflight, 1, 0,
                                           4 * mask, sw.sink.data_ptr(), sw.stream.cuda_stream), "llmi_hip_probe_stream_tiles")
            us = sw.us_per_call(enq, reps=2, steps=n_slices(ctx))
            if us < best[0]:
                best = (us, 32 * N_KV, waves, inflight, mask)
        us, wg, waves, inflight, mask = best
        gbs = 2 * ctx * KV_DIM * 2 / (us * 1e-6) / 1e9
        rows.append({"ctx": ctx, "us": round(us, 3), "GBps": round(gbs, 1), "frac_peak": round(gbs / HBM_PEAK_GBS, 4),
                     "workgroups": wg, "waves": waves, "tiles_in_flight": inflight, "stagger_mask": mask})
    return rows


DISPATCH_CTX = [96, 160, 176, 300, 700, 1024, 1500, 3000, 4097, 5000, 9000, 12345, 20000, 32768]


def dispatch_rows(sw, ctx_list):
    """What the dispatcher picks against forced alternatives, per context length: single pass, and the fused
    split path at several split counts; same timing method as the per-context figures. Every plan -- the automatic
    one and each forced one -- is timed equally often (two rounds over all plans, three batches of graph replays
    each) and judged by the MEDIAN of its six batches."""
    B = sw.B
    rows = []
    for ctx in ctx_list:
        def timed(**over):
            return sw.us_per_call(lambda f, n: sw.enqueue([ctx], f, n, **over), steps=n_slices(ctx), stat="all")
        plans = {"auto": {}}
        if ctx <= 1024:
            plans["single"] = dict(force_path=B.PATH_SINGLE_PASS)
        tiles = (ctx + 15) // 16
        for sp in (4, 8, 16, 32, 64):
            if sp <= tiles:
                plans["split%d" % sp] = dict(force_path=B.PATH_SPLIT_FUSED, num_splits=sp)
        timed()  # the first graph timed on a context's slices runs up to a microsecond per call slow: discard one
        samples = {name: [] for name in plans}
        for _ in range(2):
            for name, over in plans.items():
                samples[name] += timed(**over)
        med = {name: sorted(v)[len(v) // 2] for name, v in samples.items()}
        auto = med.pop("auto")
        best = min(med, key=med.get)
        p = sw.plan(ctx)
        rows.append({"ctx": ctx, "auto_us": round(auto, 2), "auto_plan": "path%d S=%d W=%d" % (p.path, p.num_splits, p.waves_per_group),
                     "best_forced": best, "best_forced_us": round(med[best], 2), "auto_over_best": round(auto / med[best], 3),
                     "forced_us": {k2: round(v2, 2) for k2, v2 in med.items()}})
    return rows


def per_ctx_rows(sw, ctx_list, replays):
    rows = []
    for ctx in ctx_list:
        us = sw.us_per_call(lambda f, n: sw.enqueue([ctx], f, n), reps=3, replays=replays, steps=n_slices(ctx))
        gbs = algorithmic_bytes(ctx, sw.n_q) / (us * 1e-6) / 1e9
        p = sw.plan(ctx)
        rows.append({"ctx": ctx, "us_per_layer": round(us, 3), "GBps": round(gbs, 1), "frac_peak": round(gbs / HBM_PEAK_GBS, 4),
                     "path": p.path, "splits": p.num_splits, "waves": p.waves_per_group})
    return rows


def run_calibrate_hbm(args):
    """A plain copy kernel of known traffic, for scaling the FETCH_SIZE / WRITE_SIZE counters:
    rocprofv3 --pmc FETCH_SIZE --kernel-trace -- python3 bench.py --calibrate-hbm"""
    import torch
    from llminfer_amd import _binding as B
    gib = 1 << 30
    src = torch.ones(gib // 4, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(6):
        B.check(B.lib().llmi_hip_probe_copy(src.data_ptr(), dst.data_ptr(), gib, torch.cuda.current_stream().cuda_stream), "copy")
    torch.cuda.synchronize()
    print(json.dumps({"metric": "calibration copy", "kernel": "copy_kernel", "dispatches": 6, "bytes_read_per_dispatch": gib,
                      "bytes_written_per_dispatch": gib, "ok": bool(torch.equal(src[:1024], dst[:1024]))}))
    return 0


def run_stack_timeline(args, ctx):
    """Where a layer's time goes inside the resident launch (llmi_hip_mha_decode_append_stack): needs a build of the
    library with the phase stamps compiled in,

        python -m llminfer_amd.build --define LLMI_STACK_STAMPS=1 --only mha_stack.hip --output /tmp/libllmi_stamps.so
        LLMI_HIP_LIBRARY=/tmp/libllmi_stamps.so python bench.py --stack-timeline --ctx 4096

    which writes the 100 MHz clock at the phases of four layers (16 .. 19 of 36) into the workspace, 4 MiB in; this mode runs
    the launch once after three warm-up launches and condenses the stamps. Times in us (ticks of 10 ns)."""
    import numpy as np
    import torch
    from llminfer_amd import _binding as B
    from llminfer_amd import ops
    dev = torch.device("cuda:0")
    L, n_q, D = 36, args.heads, HEAD_DIM
    msl, pos, dim = ctx + 8, ctx, n_q * D
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)

    def rnd(*shape, norm=True):
        x = torch.randn(shape, generator=gen, device=dev)
        if norm:
            x = x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True))
        return x.to(torch.bfloat16)

    k, v = rnd(L * N_KV * msl, D).reshape(-1), rnd(L * N_KV * msl, D).reshape(-1)
    q, kn, vn = rnd(L * n_q, D, norm=False).reshape(-1), rnd(L * N_KV, D, norm=False).reshape(-1), rnd(L * N_KV, D, norm=False).reshape(-1)
    w = (1 + 0.02 * torch.randn(L * 2 * D, generator=gen, device=dev)).to(torch.bfloat16)
    out = torch.zeros(L * dim, dtype=torch.bfloat16, device=dev)
    sin_d, cos_d = ops.sincos_table(D, msl, dev)
    ws = torch.zeros(max(ops.workspace_bytes(n_q, D, msl), 6 << 20) // 4, dtype=torch.float32, device=dev)
    side = ops.workspace_side(ws)
    kw = dict(layer_id=0, pos=pos, kv_dim=KV_DIM, kv_mul=n_q // N_KV, head_num=n_q, head_dim=D, max_seq_len=msl,
              kv_layout=B.KV_LAYOUT_HEAD_MAJOR, workspace_side=side)

    def run():
        n = ops.mha_decode_append_stack(q, kn, vn, w, sin_d, cos_d, k, v, out, ws, layer_count=L, query_stride=dim, key_new_stride=KV_DIM,
                                        value_new_stride=KV_DIM, norm_weight_stride=2 * D, output_stride=dim, **kw)
        torch.cuda.synchronize()
        return n

    for _ in range(3):
        run()
    plan = ops.mha_plan(ops.make_mha_args(q, k, v, out, ws, **dict(kw, pos=pos - 1)))  # (the stack plans for the cached positions)
    pad = ((-ws.data_ptr()) & 16383) if side else 0  # (the by-side layout starts on the next 16 KiB boundary)
    first = (pad + (4 << 20)) // 4
    ws[first:].zero_()
    torch.cuda.synchronize()
    if run() != 1:
        print("bench.py: the one-launch form does not apply to this shape", file=sys.stderr)
        return 1
    S = plan.num_splits
    grid = N_KV * S
    st = ws[first:first + 4 * grid * 16].cpu().numpy().view(np.uint32).reshape(4, grid, 16).astype(np.int64)
    if not st.any():
        print("bench.py: no stamps found: build the library with --define LLMI_STACK_STAMPS=1 (see --help)", file=sys.stderr)
        return 1
    split = np.arange(grid) // N_KV
    group = n_q // N_KV
    merging = (split >= S - group) if S >= group else (split == S - 1)

    def stats(x):
        return {"min": round(float(x.min()) / 100, 2), "median": round(float(np.median(x)) / 100, 2), "max": round(float(x.max()) / 100, 2)}

    layers = []
    for l in range(1, 4):
        t0 = st[l - 1, merging, 6].max()  # the last tag of the layer before
        layers.append({
            "layer": 16 + l,
            "tags_seen_after_last_tag": stats(st[l, :, 0] - t0),
            "operands_landed_after_tags_seen": stats(st[l, :, 1] - st[l, :, 0]),
            "tiles_done_after_operands": stats(st[l, :, 8:12] - st[l, :, 1:2]),
            "handed_over_after_tiles_done": stats(st[l, :, 3] - st[l, :, 2]),
            "merging_records_in_after_own_hand_over": stats(st[l, merging, 4] - st[l, merging, 3]),
            "merging_rows_read_back_after_records": stats(st[l, merging, 5] - st[l, merging, 4]),
            "merging_tag_out_after_read_back": stats(st[l, merging, 6] - st[l, merging, 5]),
            "layer_period": round(float(st[l, merging, 6].max() - t0) / 100, 2),
        })
    print(json.dumps({"metric": "phases of a layer inside the resident launch, us (100 MHz clock stamps of one launch)", "n_gpus": 1,
                      "config": {"workload": "36 layers, %d Q / 8 KV heads, ctx %d + 1, %d splits; every figure over all %d workgroups (merging_*: "
                                             "over the %d that merge a head)" % (n_q, ctx, S, grid, int(merging.sum()))},
                      "note": "a stamp is a store: wavefront 0's own stamps add up to 0.4 us to its tile phase (its next tile wait also waits "
                              "for the stamp's acknowledgement); the other wavefronts' tile times (tiles_done_after_operands covers all four) "
                              "are undisturbed",
                      "layers": layers}))
    return 0


STREAM_MODES = ["registers, linear", "LDS-DMA, linear", "LDS-DMA, K swizzled (the decode kernel's requests)",
                "LDS-DMA, K swizzled, pause after every tile"]


def run_stream_variants(args, ctx_list):
    """The decode kernel's K/V stream without its arithmetic, one feature at a time (llmi_hip_probe_stream_tiles), on the decode
    kernel's own grid of 32 splits x 8 KV heads, next to the decode kernel itself: which feature of the request pattern costs
    bandwidth, in both cache layouts. Same graph-replay timing and rotating KV slices as the headline figures."""
    import torch
    from llminfer_amd import _binding as B
    from llminfer_amd import ops
    n_q = args.heads
    waves, inflight = (8, 1) if n_q // N_KV >= 8 else (4, 2)
    probe = B.lib().llmi_hip_probe_stream_tiles
    rows = []
    for layout in (1, 0):
        sw = Sweep(ctx_list, n_q, layout)
        for ctx in ctx_list:
            decode_us = sw.us_per_call(lambda f, n: sw.enqueue([ctx], f, n), reps=3, replays=40, steps=n_slices(ctx))
            row = {"ctx": ctx, "layout": "head-major" if layout == 1 else "position-major", "splits": 32, "waves": waves,
                   "tiles_in_flight": inflight, "decode_us": round(decode_us, 2), "variants": []}
            for mode, pause, stagger in ((0, 0, 0), (1, 0, 0), (2, 0, 0), (3, 4, 0), (3, 8, 0), (3, 16, 0), (0, 0, 2), (2, 0, 2), (2, 0, 1), (2, 0, 4 * 31), (2, 0, 2 + 4 * 31)):
                def enq(first, n):
                    for st in range(first, first + n):
                        off = sw.regions[(ctx, st % n_slices(ctx))] * 2
                        B.check(probe(sw.k.data_ptr() + off, sw.v.data_ptr() + off, ctx, N_KV, layout, 32, waves, inflight, mode, pause,
                                      stagger, sw.sink.data_ptr(), sw.stream.cuda_stream), "llmi_hip_probe_stream_tiles")
                us = sw.us_per_call(enq, reps=3, replays=40, steps=n_slices(ctx))
                row["variants"].append({"mode": STREAM_MODES[mode] + (" (%d x 64 clocks)" % pause if mode == 3 else "") +
                                                (", staggered walk (mask %d)" % (3 if stagger & 1 else stagger >> 2) if stagger & ~2 else "") +
                                                (", splits fastest in the grid" if stagger & 2 else ""),
                                        "us": round(us, 2), "TBps": round(2 * ctx * KV_DIM * 2 / us / 1e6, 3)})
            rows.append(row)
        del sw
        torch.cuda.empty_cache()
    print(json.dumps({"metric": "K/V stream variants next to the decode kernel, us per launch (graph replays, best of 3 batches)", "n_gpus": 1,
                      "config": {"workload": "%d Q / 8 KV heads; K and V rows of one call read once and thrown away by a kernel with the decode "
                                             "kernel's grid and tile deal" % n_q}, "rows": rows}))
    return 0


def run_placement(args):
    """Where the workgroups of a 128 / 256 / 512-workgroup launch with a decode workgroup's footprint land."""
    import collections
    import torch
    from llminfer_amd import _binding as B
    ids = torch.zeros(2 * 512, dtype=torch.int32, device="cuda:0")
    rows = []
    for wgs in (128, 256, 512):
        for exclusive in (0, 1):
            ids.zero_()
            B.check(B.diag_lib().llmi_diag_placement(wgs, exclusive, ids.data_ptr(), torch.cuda.current_stream().cuda_stream), "placement probe")
            torch.cuda.synchronize()
            a = ids[:2 * wgs].cpu().numpy().astype("uint32").reshape(-1, 2)
            per_cu = collections.Counter((int(x), (int(h) >> 8) & 0xFF) for x, h in a)
            per_xcd = collections.Counter(int(x) for x in a[:, 0])
            rows.append({"workgroups": wgs, "lds_kib": 84 if exclusive else 66, "distinct_cus": len(per_cu), "max_per_cu": max(per_cu.values()),
                         "per_xcd": [per_xcd.get(i, 0) for i in range(8)]})
    print(json.dumps({"metric": "placement of workgroups with a decode workgroup's footprint (256 threads, 66 or 84 KiB of LDS, 5 us each)",
                      "n_gpus": 1, "rows": rows}))
    return 0


def run_handover_probe(args):
    """How a 4-byte value stored by one workgroup becomes visible to a polling workgroup on the same XCD and
    on another one, for every pair of store / load cache policies."""
    import torch
    from llminfer_amd import _binding as B
    names = ["plain", "sc0", "sc1", "sc0 sc1", "nt"]
    line = torch.zeros(1024, dtype=torch.int32, device="cuda:0")
    res_d = torch.zeros(8, dtype=torch.int32, device="cuda:0")
    rows = []
    for place, reader in (("same XCD", 8), ("next XCD", 9)):
        for precache in (1, 0):
            for st in range(5):
                for ld in range(5):
                    reps = []
                    for _ in range(3):
                        B.check(B.diag_lib().llmi_diag_handover(st, ld, 0, reader, precache, line.data_ptr(), res_d.data_ptr(),
                                                               torch.cuda.current_stream().cuda_stream), "handover probe")
                        torch.cuda.synchronize()
                        r = res_d.cpu().numpy()
                        reps.append({"seen": int(r[0]), "polls": int(r[1]), "ns": int(r[2]), "xcc_reader": int(r[3]), "xcc_writer": int(r[4])})
                    rows.append({"placement": place, "precache": precache, "store": names[st], "load": names[ld], "runs": reps})
    print(json.dumps({"metric": "hand-over probe: store policy x load policy, reader polls until it sees the writer's value "
                                "(writer waits 2 us before storing; 4000 polls at most)", "rows": rows}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--ctx", type=str, default=",".join(map(str, DEFAULT_CTX)))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--plain-workspace", action="store_true",
                    help="skip llmi_hip_mha_workspace_side: the fused combine's plain workspace layout, wherever it happens to lie")
    ap.add_argument("--no-extras", action="store_true",
                    help="headline sweep only: skip the stream floor, the position-major layout, BASELINE configs 4 and 5 "
                         "and the dispatch check that the default run appends to its JSON line")
    ap.add_argument("--sweep-only", action="store_true",
                    help="like --no-extras, and no per-length replays either: every launch of the process is part of the sweep")
    ap.add_argument("--dispatch-check", action="store_true",
                    help="time the automatic plan against forced single-pass / split plans at every --ctx")
    ap.add_argument("--stream-floor", action="store_true",
                    help="time a kernel that only reads the same K/V bytes, next to the decode kernel, at every --ctx")
    ap.add_argument("--stack-timeline", action="store_true",
                    help="phases of a layer inside the resident launch from in-kernel clock stamps; needs a library built with "
                         "--define LLMI_STACK_STAMPS=1 (LLMI_HIP_LIBRARY), see run_stack_timeline")
    ap.add_argument("--stream-variants", action="store_true",
                    help="time the decode kernel's K/V stream without its arithmetic, one feature of the request pattern at a time, "
                         "in both cache layouts, at every --ctx")
    ap.add_argument("--calibrate-hbm", action="store_true", help="run the copy kernel of known traffic (for rocprofv3 --pmc)")
    ap.add_argument("--handover-probe", action="store_true", help="store/load cache-policy visibility probe between two workgroups")
    ap.add_argument("--placement", action="store_true", help="which XCD and CU the workgroups of a 128/256/512-workgroup launch land on")
    ap.add_argument("--layout", type=int, default=1, help="1 = head-major (default), 0 = position-major")
    ap.add_argument("--heads", type=int, default=N_Q, help="query heads (32 = Qwen3-4B, 64 = Qwen3-32B head layout)")
    ap.add_argument("--stack", type=int, default=0, metavar="LAYERS",
                    help="instead of the sweep: LAYERS layers of (QK-Norm + RoPE + append, attention) at --ctx (one "
                         "value) + 1 new token, captured into one HIP graph; reports us per token")
    ap.add_argument("--gemv", choices=sorted(GEMV_SHAPES), default=None,
                    help="time one of the GEMVs around the attention instead (Qwen3-4B shapes)")
    ap.add_argument("--stack-follow-pos", action="store_true",
                    help="with --stack: capture once for every position (kernels read it from device memory)")
    ap.add_argument("--stack-mode", type=int, default=2,
                    help="with --stack: 5 = one resident launch for all layers (same work as 2); 4 = whole attention block in two launches per layer (QKV GEMV, attention + o_proj + "
                         "residual in one); 3 = the block in three launches (QKV GEMV, attention, o_proj + residual); "
                         "2 = norm/rope/append fused into the attention launch (default), "
                         "1 = separate kernel before attention (the reference's sequence)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus %d refused): decode attention at batch 1 "
              "has no multi-GPU part here." % args.gpus, file=sys.stderr)
        return 2
    if args.steps < 1 or args.warmup < 0:
        print("bench.py: --steps must be positive, --warmup non-negative", file=sys.stderr)
        return 2
    ctx_list = [int(c) for c in args.ctx.split(",")]
    n_q = args.heads

    import torch
    from llminfer_amd import _binding as B
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    B.lib()  # fail loudly if the HIP library is not built
    torch.cuda.set_device(torch.device("cuda:0"))

    if args.calibrate_hbm:
        return run_calibrate_hbm(args)
    if args.handover_probe:
        return run_handover_probe(args)
    if args.placement:
        return run_placement(args)
    if args.gemv:
        return run_gemv(args)
    if args.stack:
        return run_stack(args, ctx_list[0])
    if args.stream_variants:
        return run_stream_variants(args, ctx_list)
    if args.stack_timeline:
        return run_stack_timeline(args, ctx_list[0])

    sw = Sweep(ctx_list, n_q, args.layout, args.plain_workspace)
    layout_name = "head-major" if args.layout == 1 else "position-major"

    if args.dispatch_check:
        rows = dispatch_rows(sw, ctx_list)
        print(json.dumps({"metric": "dispatch check: auto plan against forced paths, us per layer call", "n_gpus": 1,
                          "config": {"workload": "%d Q / 8 KV heads, %s layout" % (n_q, layout_name)},
                          "rows": rows, "worst_auto_over_best": max(r["auto_over_best"] for r in rows)}))
        return 0
    if args.stream_floor:
        floor = stream_floor(sw, ctx_list)
        mine = per_ctx_rows(sw, ctx_list, 40)
        rows = [dict(f, decode_us=m["us_per_layer"], decode_frac_peak=m["frac_peak"], decode_minus_floor_us=round(m["us_per_layer"] - f["us"], 3))
                for f, m in zip(floor, mine)]
        print(json.dumps({"metric": "stream-only floor next to the decode kernel, us per launch (graph replays)", "n_gpus": 1,
                          "config": {"workload": "K and V rows of one call (%d Q / 8 KV heads, %s) read once and thrown away; best of %d "
                                                 "launch shapes" % (n_q, layout_name, len(FLOOR_CONFIGS))},
                          "rows": rows}))
        return 0

    # ---- the timed region: EXACTLY --steps steps of the whole sweep, after --warmup untimed ones ----------
    # A graph holds SWEEP_GRAPH_STEPS steps (the KV slices in turn, five times round: 240 launches, about what a decode
    # step of a 36-layer model puts into its graph; between two replays of a graph the device idles for some
    # microseconds, which short graphs would charge to the kernel); a second, shorter graph holds the remainder.
    def sweep_enqueue(first, n):
        sw.enqueue(ctx_list, first, n)

    g_full = sw.capture(sweep_enqueue, SWEEP_GRAPH_STEPS)
    rem_graphs = {}

    def replays_for(k):
        full, rem = divmod(k, SWEEP_GRAPH_STEPS)
        seq = [(g_full, full)] if full else []
        if rem:
            if rem not in rem_graphs:
                rem_graphs[rem] = sw.capture(sweep_enqueue, rem)
            seq.append((rem_graphs[rem], 1))
        return seq

    timed_seq = replays_for(args.steps)  # (captured before the clock starts)
    warm_seq = replays_for(args.warmup) if args.warmup else []
    # Set-up, like the arena fill: a fifth of a second of the same work lets the clocks settle (a cold device
    # runs the first milliseconds 5-8 % slow), so that short --steps / --warmup values measure the steady state
    # too. These replays are neither warm-up steps nor timed.
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < 0.2:
        sw.time_replays([(g_full, 4)])
    if warm_seq:
        sw.time_replays(warm_seq)
    ms = sw.time_replays(timed_seq)
    steps = args.steps
    ms_per_step = ms / steps
    step_bytes = sum(algorithmic_bytes(c, n_q) for c in ctx_list)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    launches_per_step = len(ctx_list)  # every call of the sweep is one launch of the decode kernel

    # ---- the same sweep again for at least half a second: median over batches (a short --steps leaves a
    # timed region of a millisecond or two, which a machine hiccup can move) ---------------------------
    batch_ms = []
    t_long = time.perf_counter()
    while len(batch_ms) < 5 or (time.perf_counter() - t_long < 0.5 and len(batch_ms) < 400):
        batch_ms.append(sw.time_replays([(g_full, 2)]) / (2 * SWEEP_GRAPH_STEPS))
    batch_ms.sort()
    median_ms = batch_ms[len(batch_ms) // 2]

    # (--sweep-only: nothing but the sweep is launched, every length equally often -- what the HBM counters are taken on)
    per_ctx = [] if args.sweep_only else per_ctx_rows(sw, ctx_list, 40)
    avg_launch_us = ms_per_step * 1e3 / launches_per_step
    avg_launch_bytes = step_bytes / launches_per_step
    achieved = avg_launch_bytes / (avg_launch_us * 1e-6) / 1e9
    result = {
        "metric": "GQA decode attn us/layer + HBM GB/s (% peak), Qwen3-4B shape, ctx 1K-32K",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s layer shape (%d Q / 8 KV heads, head_dim 128), batch 1, one decode-"
                               "attention layer call per context in %s per step, bf16 KV cache, %s layout, "
                               "HIP-graph replays over %d rotating KV slices per context (per-context figures: over at "
                               "least 512 MiB of slices from 1024 positions up, so no length replays out of the 256 MB Infinity Cache)"
                               % ("Qwen3-4B" if n_q == 32 else "Qwen3-32B-heads" if n_q == 64 else "custom", n_q,
                                  ctx_list, layout_name, SLICES),
                   "ctx": ctx_list, "bytes_per_step": step_bytes, "kv_layout": args.layout,
                   "workspace_side": "0x%x" % (sw.side & 0xffffffff)},
        "timed_region_s": round(ms * 1e-3, 6),
        "long_run": {"seconds": round(sum(batch_ms) * 2 * SWEEP_GRAPH_STEPS * 1e-3, 3), "batches": len(batch_ms), "steps_per_batch": 2 * SWEEP_GRAPH_STEPS,
                     "ms_per_step_median": round(median_ms, 6), "value_median": round(step_bytes / (median_ms * 1e-3) / 1e9, 1),
                     "ms_per_step_p10": round(batch_ms[len(batch_ms) // 10], 6), "ms_per_step_p90": round(batch_ms[len(batch_ms) * 9 // 10], 6)},
        "us_per_layer_mean": round(avg_launch_us, 3),
        "per_ctx_stat": "per_ctx, position_major, stream_floor and cfg5 figures: best of 3 (floor: 2) batches of graph replays of one "
                        "length alone; dispatch_check: median of 6 batches per plan; value, ms_per_step and roofline: the timed "
                        "region itself, nothing picked",
        "per_ctx": per_ctx,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(ctx_list) if n_q == N_Q and args.layout == 1 else None,
                     "kernel": "mha_decode_kernel", "launches": steps * launches_per_step,
                     "avg_launch_us": round(avg_launch_us, 3), "avg_launch_bytes": int(avg_launch_bytes)},
    }

    if not args.no_extras and not args.sweep_only:
        # What one launch can reach on this machine with the same bytes: the stream-only floor per context.
        floor = stream_floor(sw, ctx_list)
        for row, f in zip(per_ctx, floor):
            row["stream_floor_us"] = f["us"]
            row["stream_floor_frac_peak"] = f["frac_peak"]
            row["floor_ratio"] = round(f["us"] / row["us_per_layer"], 3)  # stream-only floor / decode kernel: 1 = at the floor
        result["stream_floor"] = floor
        del sw
        torch.cuda.empty_cache()
        if n_q == N_Q and args.layout == 1:
            # the reference's own cache layout (what a maintainer gets who changes nothing but the registry arm)
            sw_pm = Sweep(ctx_list, n_q, 0)
            result["position_major"] = per_ctx_rows(sw_pm, ctx_list, 40)
            for row, f in zip(result["position_major"], stream_floor(sw_pm, ctx_list)):  # the same pieces, read and thrown away
                row["stream_floor_us"] = f["us"]
                row["floor_ratio"] = round(f["us"] / row["us_per_layer"], 3)
            del sw_pm
            torch.cuda.empty_cache()
            # the dispatch against forced plans at lengths either side of the threshold, powers of two and not
            sw_d = Sweep(DISPATCH_CTX, n_q, 1)
            rows = dispatch_rows(sw_d, DISPATCH_CTX)
            result["dispatch_check"] = {"stat": "median of 6 batches per plan, automatic and forced plans timed equally often",
                                        "worst_auto_over_best": max(r["auto_over_best"] for r in rows),
                                        "rows": [{k2: r[k2] for k2 in ("ctx", "auto_us", "auto_plan", "best_forced", "best_forced_us", "auto_over_best")}
                                                 for r in rows]}
            del sw_d
            torch.cuda.empty_cache()
            # BASELINE config 5: 64 Q / 8 KV heads at ctx 131072 (512 MiB of K and V per call)
            sw5 = Sweep([131072], 64, 1)
            r5 = per_ctx_rows(sw5, [131072], 40)[0]
            f5 = stream_floor(sw5, [131072], FLOOR_CONFIGS[:4])[0]
            result["cfg5"] = dict(r5, workload="64 Q / 8 KV heads, ctx 131072, head-major, graph replays over %d KV slices" % SLICES,
                                  stream_floor_us=f5["us"], floor_ratio=round(f5["us"] / r5["us_per_layer"], 3))
            del sw5
            torch.cuda.empty_cache()
            # BASELINE config 4: 36 layers at ctx 4096 + 1 new token, fused QK-Norm + RoPE + append, one HIP graph per token
            ns = argparse.Namespace(stack=36, heads=32, layout=1, stack_mode=5, stack_follow_pos=False, steps=200, warmup=20)
            r4 = stack_result(ns, 4096)
            ns.stack_mode = 2
            r4b = stack_result(ns, 4096)
            if r4 is not None and r4b is not None:
                result["cfg4_stack"] = {"us_per_token": r4["value"], "us_per_layer": r4["us_per_layer"],
                                        "frac_peak": r4["roofline"]["frac"], "GBps": r4["roofline"]["achieved"],
                                        "workload": r4["config"]["workload"],
                                        "one_launch_per_layer": {"us_per_token": r4b["value"], "us_per_layer": r4b["us_per_layer"],
                                                                 "frac_peak": r4b["roofline"]["frac"],
                                                                 "workload": r4b["config"]["workload"]}}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(ctx_list, n_q=n_q)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
