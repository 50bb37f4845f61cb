"""The library's measurement aids (no counterpart in the reference): they must not change results, and what they report must
be consistent with itself.

  eisen_hip_attention_timeline    the hd-64 attention kernels drop time stamps; outputs stay the bits of the plain kernels
  eisen_hip_attention_ablation    leaves part of the backward kernels out (results wrong by construction); part 0 restores them
  eisen_hip_attention_tile_model  model of the dK/dV tile loop: positive times, more parts never faster than the MFMAs alone
  eisen_hip_mfma_ceiling          below the published peak, above half of it
"""
import numpy as np
import pytest

from eisen_amd import hip
from eisen_amd.lib import EisenHipError
from tests import gen
from tests.gpu_util import ctx  # noqa: F401

pytestmark = pytest.mark.gpu
BF16 = hip.BF16


def _attention(ctx, B, S, Hq, Hkv, hd, run):
    sd = 1.0 / np.sqrt(hd)
    q, do = gen.normal(910, (B, S, Hq, hd), sd), gen.normal(911, (B, S, Hq, hd), sd)
    k, v = gen.normal(912, (B, S, Hkv, hd), sd), gen.normal(913, (B, S, Hkv, hd), sd)
    dq_, dk_, dv_, ddo = (ctx.upload(t, BF16) for t in (q, k, v, do))
    out, lse = ctx.malloc(q.size * 2), ctx.malloc(B * Hq * S * 4)
    gq, gk, gv = ctx.malloc(q.size * 2), ctx.malloc(k.size * 2), ctx.malloc(k.size * 2)
    scale = float(1.0 / np.sqrt(hd))
    results = []
    for _ in range(run):
        ctx.attention_forward(dq_, dk_, dv_, out, lse, BF16, B, S, Hq, Hkv, hd, scale, True)
        ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, BF16, B, S, Hq, Hkv, hd, scale, True)
        ctx.sync()
        results.append([ctx.download(b, n, np.uint16).copy() for b, n in ((out, q.size), (gq, q.size), (gk, k.size), (gv, k.size))])
        yield results[-1]
    for b in (dq_, dk_, dv_, ddo, out, lse, gq, gk, gv):
        b.free()


def test_timeline_leaves_the_results_alone_and_its_stamps_are_in_order(ctx):
    B, S, Hq, Hkv, hd = 4, 512, 16, 4, 64          # 16 query blocks x 16 (batch, KV head): 256 blocks of four waves; 128 key-block pairs
    waves = 1024
    stamps = ctx.malloc(3 * waves * 16 * 8, zero=True)
    runs = _attention(ctx, B, S, Hq, Hkv, hd, 2)
    plain = next(runs)
    ctx.attention_timeline(stamps, waves)
    timed = next(runs)
    ctx.attention_timeline(None, 0)
    for a, b, name in zip(plain, timed, ("O", "dQ", "dK", "dV")):
        assert np.array_equal(a, b), f"{name} differs when the kernels drop time stamps"
    t = ctx.download(stamps, (3, waves, 8, 2), np.int64)
    for kern, (name, n_waves) in enumerate((("forward", 1024), ("dQ", 1024), ("dK/dV", 512))):
        w = t[kern, :, :, 0]
        live = w[:, 0] > 0
        assert live.sum() == n_waves, (name, int(live.sum()))
        w = w[live]
        assert (w[:, 1] >= w[:, 0]).all() and (w[:, 2] >= w[:, 1]).all() and (w[:, 3] >= w[:, 2]).all(), f"{name}: stamps out of order"
        second = w[:, 6] > 0
        assert (w[second, 4] >= w[second, 3]).all() and (w[second, 5] >= w[second, 4]).all() and (w[second, 6] >= w[second, 5]).all()
        span_us = (np.where(second, w[:, 6], w[:, 3]).max() - w[:, 0].min()) * 1e-2
        assert 1.0 < span_us < 1000.0, (name, span_us)
    stamps.free()
    with pytest.raises(EisenHipError):
        ctx.attention_timeline(None, 5)        # a wave count without a buffer


def test_ablation_zero_restores_the_kernels(ctx):
    B, S, Hq, Hkv, hd = 2, 256, 8, 2, 64
    runs = _attention(ctx, B, S, Hq, Hkv, hd, 3)
    plain = next(runs)
    ctx.attention_ablation(5)                   # softmax arithmetic left out: wrong by construction
    wrong = next(runs)
    ctx.attention_ablation(0)
    again = next(runs)
    assert not np.array_equal(plain[1], wrong[1]), "the ablation run was expected to differ"
    for a, b in zip(plain, again):
        assert np.array_equal(a, b)
    with pytest.raises(EisenHipError):
        ctx.attention_ablation(7)


def test_tile_model_and_mfma_ceiling_report_sane_figures(ctx):
    mfma = ctx.attention_tile_model(1, 2, 1000)
    everything = ctx.attention_tile_model(15, 2, 1000)
    loads = ctx.attention_tile_model(8, 2, 1000)
    # 16 MFMAs of 32 cycles per tile and SIMD: 213 ns at the 2.4 GHz boost clock, never less
    assert 213.0 <= mfma < 2000.0, mfma
    assert everything >= 0.9 * mfma and 20.0 < loads < 2000.0, (mfma, everything, loads)
    with pytest.raises(EisenHipError):
        ctx.attention_tile_model(2, 2, 1000)
    # the one-pass tile: 16 + 4 MFMAs' worth of matrix time, never less than 266 ns at the boost clock
    one_pass = ctx.attention_tile_model(32, 2, 1000)
    assert 266.0 <= one_pass < 3000.0 and ctx.attention_tile_model(16, 2, 1000) >= 0.9 * one_pass, one_pass
    d_us, sum_us = ctx.attention_onepass_parts(4 * 1024, 1024, 128)
    assert 0.5 < d_us < 500.0 and 0.5 < sum_us < 500.0, (d_us, sum_us)
    with pytest.raises(EisenHipError):
        ctx.attention_onepass_parts(1000, 1024, 128)
    ceiling = ctx.mfma_ceiling(0, 5000)
    assert 1250.0 < ceiling < 2500.0, ceiling
    on_random_operands = ctx.mfma_ceiling(16, 5000, random_operands=True)
    assert 900.0 < on_random_operands < 2500.0, on_random_operands
