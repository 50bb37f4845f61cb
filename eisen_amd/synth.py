"""Seeded synthetic inputs (token streams, N(0, std) weights) shared by the tests, the smoke run and bench.py.

Everything derives from numpy's PCG64 (`np.random.default_rng(seed)`), so the oracle and the
GPU path regenerate identical inputs on any machine with the same numpy.
"""
import numpy as np


def rng(seed):
    return np.random.default_rng(seed)


def normal(seed, shape, std=1.0):
    return (rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def uniform_ids(seed, shape, vocab):
    return rng(seed).integers(0, vocab, size=shape, dtype=np.int64)


def zipf_ids(seed, shape, vocab, s=1.1):
    """Token ids with P(rank r) ~ 1/r^s over [0, vocab): inverse CDF on a seeded uniform."""
    ranks = np.arange(1, vocab + 1, dtype=np.float64)
    cdf = np.cumsum(ranks ** (-s))
    cdf /= cdf[-1]
    u = rng(seed).random(size=shape)
    return np.minimum(np.searchsorted(cdf, u), vocab - 1).astype(np.int64)


def lm_batch(seed, mb, seq, vocab, dist="uniform"):
    """(x ids [mb, seq], targets [mb*seq]): S+1 ids per row, x = [0..S), y = [1..S]."""
    draw = zipf_ids if dist == "zipf" else uniform_ids
    stream = draw(seed, (mb, seq + 1), vocab)
    return stream[:, :-1].copy(), stream[:, 1:].reshape(-1).copy()


def lm_param_shapes(vocab, hidden, heads, kv_heads, ffn, layers, tie):
    """Parameter shapes in construction (tensor id) order."""
    hd = hidden // heads
    kv = kv_heads * hd
    shapes = [("embed", (vocab, hidden))]
    for l in range(layers):
        shapes += [(f"l{l}.norm1", (hidden,)), (f"l{l}.wq", (hidden, hidden)), (f"l{l}.wk", (hidden, kv)),
                   (f"l{l}.wv", (hidden, kv)), (f"l{l}.wo", (hidden, hidden)), (f"l{l}.norm2", (hidden,)),
                   (f"l{l}.w_gate", (hidden, ffn)), (f"l{l}.w_up", (hidden, ffn)), (f"l{l}.w_down", (ffn, hidden))]
    shapes.append(("norm_f", (hidden,)))
    if not tie:
        shapes.append(("lm_head", (hidden, vocab)))
    return shapes


def lm_weights(seed, vocab, hidden, heads, kv_heads, ffn, layers, tie, std=0.02, perturb_norm=0.0):
    """N(0, std) matrices, norm gains 1.0 (optionally perturbed so their role is visible)."""
    out = []
    for i, (name, shape) in enumerate(lm_param_shapes(vocab, hidden, heads, kv_heads, ffn, layers, tie)):
        if len(shape) == 1:
            w = np.ones(shape, np.float32)
            if perturb_norm:
                w += normal(seed * 1000 + i, shape, perturb_norm)
        else:
            w = normal(seed * 1000 + i, shape, std)
        out.append((name, w))
    return out
