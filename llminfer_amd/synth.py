"""Seeded synthetic Qwen3-shaped attention inputs (numpy, host side).

Q, K, V are drawn N(0,1) from numpy's legacy MT19937 stream (stable across
numpy versions), optionally RMS-normalised per 128-wide head vector -- the
statistics QK-Norm leaves behind -- and rounded to bf16 (round to nearest
even). Arrays hold bf16 bit patterns as uint16.
"""
import numpy as np


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    return r.astype(np.uint16)


def bf16_bits_to_f32(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def _rms_normalise(x):
    rms = np.sqrt(np.mean(np.square(x, dtype=np.float32), axis=-1, keepdims=True, dtype=np.float32))
    return (x / rms).astype(np.float32)


def make_case(seed, *, n_q, n_kv, ctx, max_seq_len=None, layers=1, layer_id=0, head_dim=128, rms_norm=True,
              fill_layers="one"):
    """One decode-attention problem in the position-major layout.

    Returns dict(q=[n_q*head_dim] u16, k/v=[layers, max_seq_len, n_kv*head_dim] u16, and the scalars).
    Only rows 0..ctx-1 of layer `layer_id` carry data unless fill_layers == "all"; the rest hold a
    bf16 NaN pattern so that any read past `pos` or of the wrong layer poisons the result.
    """
    if max_seq_len is None:
        max_seq_len = ctx
    rng = np.random.RandomState(seed)
    kv_dim = n_kv * head_dim

    def draw(shape):
        x = rng.standard_normal(size=shape).astype(np.float32)
        if rms_norm:
            x = _rms_normalise(x.reshape(-1, head_dim)).reshape(shape)
        return f32_to_bf16_bits(x)

    q = draw((n_q * head_dim,))
    k = np.full((layers, max_seq_len, kv_dim), 0x7FC0, dtype=np.uint16)
    v = np.full((layers, max_seq_len, kv_dim), 0x7FC0, dtype=np.uint16)
    which = range(layers) if fill_layers == "all" else [layer_id]
    for l in which:
        k[l, :ctx] = draw((ctx, kv_dim))
        v[l, :ctx] = draw((ctx, kv_dim))
    return dict(q=q, k=k, v=v, layer_id=layer_id, pos=ctx - 1, kv_dim=kv_dim, kv_mul=n_q // n_kv,
                head_num=n_q, head_dim=head_dim, max_seq_len=max_seq_len, layers=layers)


def to_head_major(cache, n_kv, head_dim=128):
    """[layers, max_seq_len, n_kv*head_dim] -> [layers, n_kv, max_seq_len, head_dim] (contiguous copy)."""
    layers, msl, _ = cache.shape
    return np.ascontiguousarray(cache.reshape(layers, msl, n_kv, head_dim).transpose(0, 2, 1, 3))
