"""GPU tests of llmi_hip_mha_decode_append_stack: the attention of several consecutive layers in one resident
launch, against one llmi_hip_mha_decode_append launch per layer (same bits) and against the CPU oracle; the order
between layers (a layer's query may be the previous layer's output); the bounded waits; HIP-graph replays."""
import ctypes

import numpy as np
import pytest
import torch

from llminfer_amd import _binding as B
from llminfer_amd import ops, synth

from helpers import assert_parity, from_dev_bf16, to_dev

pytestmark = pytest.mark.gpu

D = 128


class Stack:
    """`layers` seeded caches at `ctx` positions (+1 slot for the new token) and the new token's raw rows per layer."""

    def __init__(self, dev, layers, ctx, n_q=32, n_kv=8, layout=B.KV_LAYOUT_HEAD_MAJOR, seed=11, chained=False):
        self.dev, self.layers, self.ctx, self.n_q, self.n_kv, self.layout = dev, layers, ctx, n_q, n_kv, layout
        self.msl, self.pos, self.kv_dim, self.dim = ctx + 3, ctx, n_kv * D, n_q * D
        rng = np.random.RandomState(seed)
        self.k_all = np.zeros((layers, self.msl, self.kv_dim), dtype=np.uint16)
        self.v_all = np.zeros((layers, self.msl, self.kv_dim), dtype=np.uint16)
        base = synth.make_case(seed, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=self.msl)
        for l in range(layers):  # (one seeded cache rolled per layer: distinct values in every layer, cheap to make)
            self.k_all[l, :ctx] = np.roll(base["k"][0, :ctx].reshape(-1), 128 * (l + 1)).reshape(ctx, self.kv_dim)
            self.v_all[l, :ctx] = np.roll(base["v"][0, :ctx].reshape(-1), 128 * (3 * l + 2)).reshape(ctx, self.kv_dim)
            self.k_all[l, ctx:] = 0x7FC0  # NaN behind the cached positions: nothing may read them
            self.v_all[l, ctx:] = 0x7FC0
        bits = lambda *shape: synth.f32_to_bf16_bits(rng.standard_normal(shape).astype(np.float32))
        self.q_raw, self.k_new, self.v_new = bits(layers, self.dim), bits(layers, self.kv_dim), bits(layers, self.kv_dim)
        self.w = synth.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal((layers, 2 * D))).astype(np.float32))
        self.sin_d, self.cos_d = ops.sincos_table(D, self.msl, dev)
        self.chained = chained  # layer l + 1's raw query IS layer l's output (one array of layers + 1 rows)
        self.ws = torch.full((ops.workspace_bytes(n_q, D, self.msl) // 4,), float("nan"), dtype=torch.float32, device=dev)
        self.kw = dict(layer_id=0, pos=self.pos, kv_dim=self.kv_dim, kv_mul=n_q // n_kv, head_num=n_q, head_dim=D,
                       max_seq_len=self.msl, kv_layout=layout)

    def fresh(self):
        """Device copies of everything a run writes or may alias."""
        k = self.k_all if self.layout == B.KV_LAYOUT_POS_MAJOR else synth.to_head_major(self.k_all, self.n_kv)
        v = self.v_all if self.layout == B.KV_LAYOUT_POS_MAJOR else synth.to_head_major(self.v_all, self.n_kv)
        x = np.zeros((self.layers + 1, self.dim), dtype=np.uint16)
        if self.chained:
            x[0] = self.q_raw[0]
            q, out = to_dev(x.reshape(-1), self.dev), None
            out = q[self.dim:]
        else:
            q = to_dev(self.q_raw.reshape(-1), self.dev)
            out = torch.full((self.layers * self.dim,), 0x7FC0, dtype=torch.int16, device=self.dev)
        return dict(k=to_dev(k.reshape(-1), self.dev), v=to_dev(v.reshape(-1), self.dev), q=q, out=out,
                    kn=to_dev(self.k_new.reshape(-1), self.dev), vn=to_dev(self.v_new.reshape(-1), self.dev),
                    w=to_dev(self.w.reshape(-1), self.dev))

    def run_per_layer(self, t, **over):
        """One llmi_hip_mha_decode_append launch per layer, in order."""
        for l in range(self.layers):
            kw = dict(self.kw, layer_id=l, **over)
            ops.mha_decode_append(t["q"][l * self.dim:], t["kn"][l * self.kv_dim:], t["vn"][l * self.kv_dim:], t["w"][l * 2 * D:],
                                  self.sin_d, self.cos_d, t["k"], t["v"], t["out"][l * self.dim:], self.ws, **kw)
        torch.cuda.synchronize()

    def run_stack(self, t, stream=None, **over):
        n = ops.mha_decode_append_stack(t["q"], t["kn"], t["vn"], t["w"], self.sin_d, self.cos_d, t["k"], t["v"], t["out"], self.ws,
                                        layer_count=self.layers, query_stride=self.dim, key_new_stride=self.kv_dim,
                                        value_new_stride=self.kv_dim, norm_weight_stride=2 * D, output_stride=self.dim,
                                        stream=stream, **dict(self.kw, **over))
        if stream is None:
            torch.cuda.synchronize()
        return n

    def oracle_outputs(self, oracle):
        sin_o, cos_o = oracle.sincos_table(D, self.msl)
        refs = []
        for l in range(self.layers):
            k_ref, v_ref = self.k_all[l:l + 1].copy(), self.v_all[l:l + 1].copy()
            k_ref[0, self.pos] = oracle.qk_norm_rope(self.k_new[l].reshape(self.n_kv, D), self.w[l, D:], sin_o[self.pos], cos_o[self.pos]).reshape(-1)
            v_ref[0, self.pos] = self.v_new[l]
            qn = oracle.qk_norm_rope(self.q_raw[l].reshape(self.n_q, D), self.w[l, :D], sin_o[self.pos], cos_o[self.pos]).reshape(-1)
            refs.append(oracle.mha_cpu(qn, k_ref, v_ref, 0, self.pos, self.kv_dim, self.n_q // self.n_kv, self.n_q, D, self.msl))
        return refs


def timeouts():
    n = ctypes.c_uint64()
    assert B.lib().llmi_hip_poll_timeouts(ctypes.byref(n)) == 0
    return n.value


@pytest.mark.parametrize("layers,ctx,n_q,layout,over", [
    (4, 300, 32, B.KV_LAYOUT_HEAD_MAJOR, {}),
    (4, 300, 32, B.KV_LAYOUT_POS_MAJOR, {}),
    (5, 1000, 32, B.KV_LAYOUT_HEAD_MAJOR, {}),                                   # 16 splits, ragged last tile
    (3, 5003, 32, B.KV_LAYOUT_HEAD_MAJOR, {}),                                   # three tiles per wavefront and a remainder
    (3, 2500, 32, B.KV_LAYOUT_POS_MAJOR, {"num_splits": 7, "force_path": B.PATH_SPLIT_FUSED}),
    (6, 777, 16, B.KV_LAYOUT_HEAD_MAJOR, {}),                                    # groups of two heads
    (6, 640, 8, B.KV_LAYOUT_HEAD_MAJOR, {}),                                     # one query head per KV head
    (2, 9000, 24, B.KV_LAYOUT_HEAD_MAJOR, {}),                                   # groups of three heads (padded to four)
    (1, 4096, 32, B.KV_LAYOUT_HEAD_MAJOR, {}),                                   # a run of one layer
])
def test_resident_stack_equals_one_launch_per_layer(oracle, dev, layers, ctx, n_q, layout, over):
    """One resident launch for all layers against one launch per layer on the same inputs: same outputs and same
    appended cache rows, bit for bit; the outputs also against the oracle. Twice in a row on one workspace."""
    st = Stack(dev, layers, ctx, n_q=n_q, layout=layout)
    a = st.fresh()
    st.run_per_layer(a, **over)
    refs = st.oracle_outputs(oracle)
    for l in range(layers):
        assert_parity(from_dev_bf16(a["out"][l * st.dim:(l + 1) * st.dim]), refs[l], "per-layer launches, layer %d" % l)
    before = timeouts()
    for call in range(2):
        b = st.fresh()
        assert st.run_stack(b, **over) == 1
        assert torch.equal(b["out"], a["out"]), "call %d: outputs differ" % call
        assert torch.equal(b["k"], a["k"]) and torch.equal(b["v"], a["v"]), "call %d: appended rows differ" % call
    assert timeouts() == before


def test_resident_stack_qwen3_4b_36_layers_at_4096(oracle, dev):
    """BASELINE config 4 at its full size through the one-launch form: 36 layers at 4096 cached positions + 1 new token,
    32 Q / 8 KV heads, by-side workspace as an engine would set it up. Bits of the per-layer launches, oracle parity on a
    sample of layers, and replays of a captured graph with eager work in between."""
    st = Stack(dev, 36, 4096)
    side = ops.workspace_side(st.ws) or 0x55555555
    st.ws.fill_(float("nan"))
    a = st.fresh()
    st.run_per_layer(a, workspace_side=side)
    refs = st.oracle_outputs(oracle)
    for l in (0, 1, 17, 35):
        assert_parity(from_dev_bf16(a["out"][l * st.dim:(l + 1) * st.dim]), refs[l], "layer %d" % l)
    b = st.fresh()
    assert st.run_stack(b, workspace_side=side) == 1
    assert torch.equal(b["out"], a["out"]) and torch.equal(b["k"], a["k"]) and torch.equal(b["v"], a["v"])
    # captured once, replayed with the outputs wiped and other work in between
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    c = st.fresh()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(g, stream=stream):
            st.run_stack(c, stream=stream, workspace_side=side)
    for rep in range(3):
        c["out"].fill_(0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(c["out"], a["out"]), "replay %d" % rep
        torch.randn(100000, device=dev).sum().item()


@pytest.mark.parametrize("layers,ctx,layout", [(12, 2000, B.KV_LAYOUT_HEAD_MAJOR), (36, 4096, B.KV_LAYOUT_HEAD_MAJOR),
                                               (6, 900, B.KV_LAYOUT_POS_MAJOR)])
def test_resident_stack_honours_the_order_between_layers(dev, layers, ctx, layout):
    """A layer really waits for the layer before: here layer l + 1's raw query IS layer l's output (one array of
    layers + 1 rows; query = rows 0.., output = rows 1..), so every layer's result depends on the previous layer's
    being complete and visible before its query is read. One launch per layer (stream order) gives the reference bits;
    the resident launch must give the same, on a fresh array and on replays of a captured graph."""
    st = Stack(dev, layers, ctx, layout=layout, chained=True, seed=23)
    a = st.fresh()
    st.run_per_layer(a)
    assert bool(torch.isfinite(torch.from_numpy(from_dev_bf16(a["q"]))).all())
    assert len({bytes(a["q"][l * st.dim:(l + 1) * st.dim].cpu().numpy().tobytes()) for l in range(layers + 1)}) == layers + 1
    for call in range(2):
        b = st.fresh()
        assert st.run_stack(b) == 1
        assert torch.equal(b["q"], a["q"]), "call %d" % call
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    c = st.fresh()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(g, stream=stream):
            st.run_stack(c, stream=stream)
    for rep in range(3):
        c["q"][st.dim:].fill_(0)  # the outputs; row 0 is the first layer's query
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(c["q"], a["q"]), "replay %d" % rep


def test_resident_stack_gives_up_with_nan_instead_of_hanging(dev):
    """With the poll limit forced to zero every wait of the resident launch gives up at once -- a merging workgroup's
    wait for the other splits' records, and every workgroup's wait for the previous layer's tags: the launch still ends
    normally, every output of every layer is NaN (never a plausible number computed from inputs that were not ready),
    the give-ups are counted. With the limit restored and the workspace cleared the same call is right again."""
    st = Stack(dev, 5, 3000, seed=31)
    a = st.fresh()
    st.run_per_layer(a)
    before = timeouts()
    prev = B.lib().llmi_hip_set_poll_limit(0)
    try:
        b = st.fresh()
        assert st.run_stack(b) == 1
    finally:
        assert B.lib().llmi_hip_set_poll_limit(prev) == 0
    assert np.all(np.isnan(from_dev_bf16(b["out"])))
    assert timeouts() > before
    after = timeouts()
    st.ws.fill_(float("nan"))  # (records and tags of the abandoned launch may have arrived late)
    c = st.fresh()
    assert st.run_stack(c) == 1
    assert torch.equal(c["out"], a["out"]) and timeouts() == after


def test_resident_stack_falls_back_to_one_launch_per_layer(dev):
    """Shapes the resident kernel is not built for run as one launch per layer, with the same results: a single pass
    (short context), groups of eight query heads, more splits than compute units, a length at which the per-layer launches
    stagger their walk (65536 cached positions: the resident kernel walks in step and would not give their bits), a
    workspace without room for the tags."""
    for n_q, ctx, over in ((32, 100, {}), (64, 2000, {}), (32, 4096, {"num_splits": 64, "force_path": B.PATH_SPLIT_FUSED}),
                           (16, 65536, {})):
        st = Stack(dev, 3, ctx, n_q=n_q)
        a, b = st.fresh(), st.fresh()
        st.run_per_layer(a, **over)
        assert st.run_stack(b, **over) == 3
        assert torch.equal(b["out"], a["out"]) and torch.equal(b["k"], a["k"])
    st = Stack(dev, 3, 1000)
    small = 32 * 16 * 528 + 16  # the plain layout's need at 16 splits, nothing for the tags
    st.ws = st.ws[:small // 4]
    a, b = st.fresh(), st.fresh()
    st.run_per_layer(a)
    assert st.run_stack(b) == 3
    assert torch.equal(b["out"], a["out"])


def test_resident_stack_argument_checks(dev):
    st = Stack(dev, 2, 500)
    t = st.fresh()
    for bad in (dict(layer_count=0), dict(query_stride=4), dict(output_stride=12)):
        kw = dict(layer_count=2, query_stride=st.dim, key_new_stride=st.kv_dim, value_new_stride=st.kv_dim,
                  norm_weight_stride=2 * D, output_stride=st.dim)
        kw.update(bad)
        with pytest.raises(B.LlmiError):
            ops.mha_decode_append_stack(t["q"], t["kn"], t["vn"], t["w"], st.sin_d, st.cos_d, t["k"], t["v"], t["out"], st.ws,
                                        **kw, **st.kw)
    assert B.lib().llmi_hip_mha_decode_append_stack(None) == B.STATUS["NULL_POINTER"]
