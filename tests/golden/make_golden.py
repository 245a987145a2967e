#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run from the repo root: python tests/golden/make_golden.py).

The expected outputs are NOT produced by the oracle: they come from a float64 evaluation of the
attention definition with library routines (numpy einsum, scipy.special.softmax), so that the oracle
and the HIP path are both checked against numbers neither of them made. Inputs are seeded (numpy's
legacy MT19937 stream, stable by numpy's policy) and rebuilt by the loader from the recipe below, so a
fixture stores only the scalars, a SHA-256 of the input bytes (to catch generator drift) and `expected`
(fp32, rounded once from the float64 result).

The reference repository holds no usable vectors for this path (its attention test draws time-seeded
data and stores nothing), so these are this repository's own.
"""
import hashlib
import os
import sys

import numpy as np
from scipy.special import softmax

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from llminfer_amd import synth  # noqa: E402


def attention_f64(q, k, v, layer_id, pos, n_kv, kv_mul, head_dim):
    """q [n_q*d], k/v [layers, max_seq_len, n_kv*d] as float64; softmax(q K^T / sqrt(d)) V per head."""
    n_q = n_kv * kv_mul
    L = pos + 1
    qh = q.reshape(n_q, head_dim)
    kh = k[layer_id, :L].reshape(L, n_kv, head_dim)
    vh = v[layer_id, :L].reshape(L, n_kv, head_dim)
    kq = np.repeat(kh, kv_mul, axis=1)  # [L, n_q, d]: query head h uses KV head h // kv_mul
    vq = np.repeat(vh, kv_mul, axis=1)
    s = np.einsum("hd,lhd->hl", qh, kq) / np.sqrt(float(head_dim))
    p = softmax(s, axis=1)
    return np.einsum("hl,lhd->hd", p, vq).reshape(-1)


def cfg1_fp32(seed, layers, layer_id):
    """Qwen3-0.6B head layout, fp32, 256 cached + 1 new position, N(0,1) inputs."""
    rng = np.random.RandomState(seed)
    n_q, n_kv, d, msl, pos = 16, 8, 128, 512, 256
    q = rng.standard_normal(n_q * d).astype(np.float32)
    k = np.zeros((layers, msl, n_kv * d), dtype=np.float32)
    v = np.zeros((layers, msl, n_kv * d), dtype=np.float32)
    k[layer_id, :pos + 1] = rng.standard_normal((pos + 1, n_kv * d)).astype(np.float32)
    v[layer_id, :pos + 1] = rng.standard_normal((pos + 1, n_kv * d)).astype(np.float32)
    exp = attention_f64(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), layer_id, pos, n_kv,
                        n_q // n_kv, d)
    return dict(q=q, k=k, v=v, layers=layers, layer_id=layer_id, pos=pos, max_seq_len=msl, n_q=n_q, n_kv=n_kv,
                head_dim=d, expected=exp.astype(np.float32))


def bf16_case(seed, n_q, n_kv, ctx, max_seq_len, layers, layer_id):
    c = synth.make_case(seed, n_q=n_q, n_kv=n_kv, ctx=ctx, max_seq_len=max_seq_len, layers=layers,
                        layer_id=layer_id)
    qf = synth.bf16_bits_to_f32(c["q"]).astype(np.float64)
    kf = synth.bf16_bits_to_f32(np.where(c["k"] == 0x7FC0, 0, c["k"]).astype(np.uint16)).astype(np.float64)
    vf = synth.bf16_bits_to_f32(np.where(c["v"] == 0x7FC0, 0, c["v"]).astype(np.uint16)).astype(np.float64)
    exp = attention_f64(qf, kf, vf, layer_id, ctx - 1, n_kv, n_q // n_kv, 128)
    return dict(q=c["q"], k=c["k"], v=c["v"], layers=layers, layer_id=layer_id, pos=ctx - 1,
                max_seq_len=max_seq_len, n_q=n_q, n_kv=n_kv, head_dim=128, expected=exp.astype(np.float32))


# name -> (builder, arguments): the recipe of every fixture.
RECIPES = {
    "cfg1_fp32_seed1": (cfg1_fp32, (1, 1, 0)),
    "cfg1_fp32_seed1_layer2of3": (cfg1_fp32, (1, 3, 2)),
    "bf16_4b_ctx77": (bf16_case, (41, 32, 8, 77, 96, 2, 1)),
    "bf16_32b_ctx300": (bf16_case, (42, 64, 8, 300, 300, 1, 0)),
}


def input_digest(case):
    h = hashlib.sha256()
    for name in ("q", "k", "v"):
        h.update(np.ascontiguousarray(case[name]).tobytes())
    return h.hexdigest()


def rebuild_inputs(name):
    """The inputs of fixture `name`, regenerated from its recipe (used by the tests)."""
    fn, args = RECIPES[name]
    return fn(*args)


def load(name):
    """Inputs (regenerated, digest-checked) + the stored expected output."""
    stored = np.load(os.path.join(HERE, name + ".npz"))
    case = rebuild_inputs(name)
    if input_digest(case) != str(stored["input_sha256"]):
        raise RuntimeError("golden fixture %s: regenerated inputs differ from the ones it was made with" % name)
    case["expected"] = stored["expected"]
    return case


def main():
    for name, (fn, args) in RECIPES.items():
        case = fn(*args)
        scalars = {k: v for k, v in case.items() if k not in ("q", "k", "v", "expected")}
        np.savez_compressed(os.path.join(HERE, name + ".npz"), expected=case["expected"],
                            input_sha256=input_digest(case), **scalars)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
