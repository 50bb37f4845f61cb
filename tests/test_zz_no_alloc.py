"""The allocation-free attention backward (eisen_hip_attention_backward_noalloc) against the allocating entry point.

Two calls in a row on one context, the second with a smaller input, so rows of the fixed scratch array that the
first call wrote are still there when the second runs.  The kernels are the same and deterministic, so the results
must be the same bits.  Collected last: a failure here must not hide the other GPU tests.
"""
import numpy as np
import pytest

from eisen_amd import hip
from eisen_amd.lib import EisenHipError
from tests import gen
from tests.gpu_util import ctx  # noqa: F401

pytestmark = pytest.mark.gpu

BF16, F32 = hip.BF16, hip.F32


def _run_both(ctx, dtype, B, S, Hq, Hkv, hd, seed, layout_bhsd=False):
    sd = 1.0 / np.sqrt(hd)
    shape_q, shape_k = ((B, Hq, S, hd), (B, Hkv, S, hd)) if layout_bhsd else ((B, S, Hq, hd), (B, S, Hkv, hd))
    qs = ks = None
    if layout_bhsd:
        qs, ks = (Hq * S * hd, hd, S * hd), (Hkv * S * hd, hd, S * hd)
    q, do = gen.normal(seed, shape_q, sd), gen.normal(seed + 1, shape_q, sd)
    k, v = gen.normal(seed + 2, shape_k, sd), gen.normal(seed + 3, shape_k, sd)
    es = 2 if dtype == BF16 else 4
    dq_, dk_, dv_, ddo = (ctx.upload(t, dtype) for t in (q, k, v, do))
    out, lse = ctx.malloc(q.size * es), ctx.malloc(B * Hq * S * 4)
    ref = [ctx.malloc(q.size * es), ctx.malloc(k.size * es), ctx.malloc(k.size * es)]
    got = [ctx.malloc(q.size * es), ctx.malloc(k.size * es), ctx.malloc(k.size * es)]
    scale = float(1.0 / np.sqrt(hd))
    ctx.attention_forward(dq_, dk_, dv_, out, lse, dtype, B, S, Hq, Hkv, hd, scale, True, qs, ks)
    ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, *ref, dtype, B, S, Hq, Hkv, hd, scale, True, qs, ks)
    ctx.sync()
    pool_before, free_before = ctx.pool_stats(), ctx.mem_info()[0]
    ctx.attention_backward_noalloc(dq_, dk_, dv_, out, ddo, lse, *got, dtype, B, S, Hq, Hkv, hd, scale, True, qs, ks)
    ctx.sync()
    assert ctx.pool_stats() == pool_before, "the allocation-free entry point went through the pool"
    assert ctx.mem_info()[0] == free_before, "device memory in use changed during the allocation-free call"
    for name, a, b, shape in zip(("dQ", "dK", "dV"), got, ref, (shape_q, shape_k, shape_k)):
        x, y = ctx.download(a, shape, dtype), ctx.download(b, shape, dtype)
        assert np.isfinite(x).all() and np.abs(x).max() > 0, name
        assert np.array_equal(x, y), f"{name}: B{B} S{S} Hq{Hq} Hkv{Hkv} hd{hd} differs from eisen_hip_attention_backward"
    for buf in [dq_, dk_, dv_, ddo, out, lse] + ref + got:
        buf.free()


def test_attention_backward_noalloc_matches_the_allocating_entry_point(ctx):
    print("noalloc: bf16 B2 S320 Hq8 Hkv2 hd64", flush=True)
    _run_both(ctx, BF16, 2, 320, 8, 2, 64, seed=900)
    print("noalloc: bf16 B1 S100 Hq4 Hkv2 hd64 (smaller, after the larger call)", flush=True)
    _run_both(ctx, BF16, 1, 100, 4, 2, 64, seed=910)
    print("noalloc: bf16 [B,H,S,hd] B2 S96 Hq8 Hkv2 hd32; f32 B2 S37 Hq4 Hkv2 hd16", flush=True)
    _run_both(ctx, BF16, 2, 96, 8, 2, 32, seed=920, layout_bhsd=True)
    _run_both(ctx, F32, 2, 37, 4, 2, 16, seed=930)


def test_attention_backward_noalloc_first_on_a_fresh_context_asks_the_driver_for_nothing():
    """The allocation-free call as the first backward of a context of its own, on a shape larger than anything that context
    has run: no workspace has been grown and no rotary table built that it could lean on.  The context's count of requests
    to the driver (pool misses, workspace growth, tables, pinned staging) and its workspace must not move; the result must
    equal the allocating entry point's, run afterwards."""
    c2 = hip.Context(0)
    try:
        B, S, Hq, Hkv, hd = 2, 512, 8, 2, 64
        sd, scale = 1.0 / np.sqrt(hd), float(1.0 / np.sqrt(hd))
        q, do = gen.normal(950, (B, S, Hq, hd), sd), gen.normal(951, (B, S, Hq, hd), sd)
        k, v = gen.normal(952, (B, S, Hkv, hd), sd), gen.normal(953, (B, S, Hkv, hd), sd)
        dq_, dk_, dv_, ddo = (c2.upload(t, BF16) for t in (q, k, v, do))
        out, lse = c2.malloc(q.size * 2), c2.malloc(B * Hq * S * 4)
        got = [c2.malloc(q.size * 2), c2.malloc(k.size * 2), c2.malloc(k.size * 2)]
        ref = [c2.malloc(q.size * 2), c2.malloc(k.size * 2), c2.malloc(k.size * 2)]
        c2.attention_forward(dq_, dk_, dv_, out, lse, BF16, B, S, Hq, Hkv, hd, scale, True)
        c2.sync()
        before = c2.driver_allocs()
        c2.attention_backward_noalloc(dq_, dk_, dv_, out, ddo, lse, *got, BF16, B, S, Hq, Hkv, hd, scale, True)
        c2.sync()
        assert c2.driver_allocs() == before, "the allocation-free entry point asked the driver for memory"
        c2.attention_backward(dq_, dk_, dv_, out, ddo, lse, *ref, BF16, B, S, Hq, Hkv, hd, scale, True)
        assert c2.driver_allocs() == before + 1, "the allocating entry point was expected to grow the workspace once"
        for name, a, b, shape in zip(("dQ", "dK", "dV"), got, ref, (q.shape, k.shape, k.shape)):
            assert np.array_equal(c2.download(a, shape, BF16), c2.download(b, shape, BF16)), name
    finally:
        c2.close()


def test_attention_rejects_a_softmax_scale_that_is_not_positive_and_finite(ctx):
    dummy = ctx.malloc(1 << 16)
    for bad in (0.0, -0.125, float("inf"), float("nan"), 1e-40):
        with pytest.raises(EisenHipError, match="scale"):
            ctx.attention_backward(dummy, dummy, dummy, dummy, dummy, dummy, dummy, dummy, dummy, BF16, 1, 32, 2, 1, 64, bad, True)
    dummy.free()


def test_attention_backward_noalloc_rejects_shapes_beyond_its_scratch(ctx):
    dummy = ctx.malloc(4096)
    with pytest.raises(EisenHipError, match="exceeds"):
        # 2 * 1024 * 1024 rows > 2^20: refused before anything is launched, so the small buffers are never touched
        ctx.attention_backward_noalloc(dummy, dummy, dummy, dummy, dummy, dummy, dummy, dummy, dummy, BF16, 2, 1024, 1024, 1024, 64, 0.125, True)
    dummy.free()
