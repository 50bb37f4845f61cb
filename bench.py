#!/usr/bin/env python3
"""Benchmark of the training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c5|c4|c3|c2]

The headline line is config 5: the "~1.1B" Llama-style model (vocab 32000, d 2048, 16 layers, 32 query / 8 KV
heads, head_dim 64, SiLU-gated MLP 5632, untied lm_head), seq 1024, micro-batch 4, gradient accumulation 8
(32,768 tokens per optimiser step), bf16 activations and matmuls, f32 master weights and AdamW state, synthetic
Zipf(1.1) token ids, N(0, 0.02) weights.  One "step" = zero_grad, 8 x (upload ids, forward, fused cross entropy,
loss read-back, backward), gradient-norm clip, fused AdamW -- the loop of examples/train_llm.rs:386-477, the
per-micro-batch loss read-back of :450 included (the copy is queued before the backward pass and collected
after it, so reading it does not drain the device).  One departure from that loop in the headline run, stated in the
line's `config.weight_gradient_window`: the weight gradients dW = X^T dY of the 8 micro-batches are formed once per
optimizer step, as one contraction over the 32,768 tokens of the window, instead of 8 products added in f32 (the same
sums in another rounding order, equal to 1e-4); `other_configs.c5_per_pass_weight_gradients` carries the same step with
the reference's order (`--no-window`), window 0.

Prints one JSON line.  `value` is tokens/s over K timed steps (inputs resident in host memory, weights and
optimiser state resident in HBM).  `roofline` describes the kernel symbol that takes the largest share of the
step, timed with HIP events on the library's stream in one extra, instrumented step; `kernels` lists every
instrumented launch family with its achieved TFLOP/s or GB/s.  `cpu_baseline` times the CPU oracle (a
restatement of the reference's Device::Cpu path) on a bounded sample of the same architecture.  With the default
`--workload all` the line also carries `other_configs`: the same figures for config 4 (the "14M" model), config 3
(flash attention forward + backward: the MFMA utilisation of the backward) and config 2 (fused cross entropy).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from eisen_amd import synth as gen  # noqa: E402  (seeded synthetic inputs, the same the tests use)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM-side bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs, per workload and per kernel symbol as
# `symbol_of` names it; the summaries (command, calibration factors, per-kernel rows) are the files named here.
TRAFFIC_SOURCE = {"c5": "profiles/c5_step_hbm_traffic_pmc.md", "c4": "profiles/c4_step_hbm_traffic_pmc.md", "c3": "profiles/c2_c3_hbm_traffic_pmc.md", "c2": "profiles/c2_c3_hbm_traffic_pmc.md"}
MEASURED_TRAFFIC = {
    "c5": {"gemm_tn_bf16_f32out_256x256x32_window": 18263.6e6, "gemm_tn_bf16_f32out_256x256x32": 902.8e6, "gemm_nt_bf16_bf16out_256x128x64": 213.4e6},
    "c4": {"gemm_tn_bf16_f32out_128x128x64_splitk": 57.7e6, "gemm_nt_bf16_bf16out_128x128x64": 35.7e6, "gemm_nt_bf16_bf16out_256x128x64_swiglu_bwd": 101.4e6,
           "gemm_tn_bf16_f32out_64x64x32_grouped_splitk": 40.1e6, "gemm_nn_bf16_bf16out_128x128x64_splitk": 54.2e6, "gemm_nn_bf16_swiglu_256x128x32": 85.1e6},
    "c3": {"attn_bwd": 78.7e6 + 52.4e6},
    "c2": {"ce_fused_bf16": 1048.9e6},
}

CONFIGS = {
    "c5": dict(vocab=32000, hidden=2048, heads=32, kv_heads=8, ffn=5632, layers=16, tie=False, seq=1024, mb=4, accum=8,
               label="config5 ~1.1B Llama-style (852,559,872 params untied), bf16 mixed, seq 1024, micro-batch 4, accum 8"),
    "c4": dict(vocab=8192, hidden=256, heads=8, kv_heads=2, ffn=1024, layers=6, tie=True, seq=256, mb=32, accum=1,
               label="config4 ~14M Llama-style (7,802,112 params tied), bf16 mixed, seq 256, micro-batch 32"),
}


def flops_per_token(c):
    """6*P_mm + 6*L*S*d: matmul parameters incl. lm_head, causal attention fwd+bwd without recompute."""
    d, f, L, V = c["hidden"], c["ffn"], c["layers"], c["vocab"]
    dkv = c["kv_heads"] * (d // c["heads"])
    p_mm = L * (2 * d * d + 2 * d * dkv + 3 * d * f) + d * V
    return 6 * p_mm + 6 * L * c["seq"] * d


def arch(c):
    return {k: c[k] for k in ("vocab", "hidden", "heads", "kv_heads", "ffn", "layers", "tie")}


def symbol_of(name):
    """Profile entries name one launch family; families that run the same kernel symbol (the plain and the grouped
    launch of one GEMM instantiation) are one row of a rocprofv3 kernel trace and are added up here as well."""
    return name[:-len("_grouped")] if name.endswith("_grouped") else name


def by_symbol(prof):
    out = {}
    for name, e in prof.items():
        s = out.setdefault(symbol_of(name), dict(ms=0.0, launches=0, work=0.0, unit=e["unit"], families=[]))
        s["ms"] += e["ms"]
        s["launches"] += e["launches"]
        s["work"] += e["work"]
        s["families"].append(name)
    return out


def roofline_of(name, e, workload, strict=False):
    """achieved = algorithmic work of the symbol's launches / their summed duration (= work per launch / average
    launch duration, weighted over the shapes the symbol ran)."""
    table = MEASURED_TRAFFIC.get(workload, {})
    traffic = table.get(name)
    if strict and table and traffic is None:
        # not fatal (the line must still come out), but loud: a kernel was renamed or the counter runs are stale.  That every key of
        # the table still names a profile entry of the library is checked by tests/test_bench_tables.py.
        print(f"bench.py: {workload}: the dominant kernel symbol {name!r} has no row in MEASURED_TRAFFIC (table of {TRAFFIC_SOURCE.get(workload)})",
              file=sys.stderr)
    src = TRAFFIC_SOURCE.get(workload) if traffic is not None else None
    if e["unit"] == "flop":
        achieved = e["work"] / (e["ms"] * 1e-3) / 1e12
        r = dict(bound="mfma", achieved=round(achieved, 2), peak=PEAK_BF16_TFLOPS, unit="TFLOP/s", frac=round(achieved / PEAK_BF16_TFLOPS, 4))
    else:
        achieved = e["work"] / (e["ms"] * 1e-3) / 1e9
        r = dict(bound="hbm", achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s", frac=round(achieved / PEAK_HBM_GBS, 4))
    r.update(traffic=traffic, traffic_source=src, kernel=name, launches=e["launches"], avg_us=round(1e3 * e["ms"] / e["launches"], 2))
    return r


PROBES = True   # --no-probes: leave out the launches that only measure the GPU (MFMA ceilings, GEMMs by operand data), for kernel traces


def mfma_ceiling(ctx):
    if not PROBES:
        return None
    return _mfma_ceiling(ctx)


def _mfma_ceiling(ctx):
    """What this GPU sustains on nothing but bf16 MFMAs, measured now, next to the published peak the fractions use:
    operands in registers, and re-read from LDS at the ratio of a 128x128 and of a 64x64 wave tile."""
    return dict(unit="TFLOP/s", registers_only=round(ctx.mfma_ceiling(0), 1), lds_fed_128x128_wave_tile=round(ctx.mfma_ceiling(8), 1),
                lds_fed_64x64_wave_tile=round(ctx.mfma_ceiling(16), 1), lds_fed_24_reads_per_16_mfma=round(ctx.mfma_ceiling(24), 1),
                lds_fed_32_reads_per_16_mfma=round(ctx.mfma_ceiling(32), 1),
                # the same loops on operands whose bits change from MFMA to MFMA (random sign, exponent, mantissa), as a layer's
                # activations and gradients do: the clock the part holds under matrix load depends on the data
                random_operands_registers_only=round(ctx.mfma_ceiling(0, random_operands=True), 1),
                random_operands_lds_fed_128x128_wave_tile=round(ctx.mfma_ceiling(8, random_operands=True), 1),
                random_operands_lds_fed_64x64_wave_tile=round(ctx.mfma_ceiling(16, random_operands=True), 1))


def gemms_by_operand_data(ctx):
    """The step's GEMM kernels alone on the GPU at config-5 shapes, once on all-zero operands and once on N(0,1) operands (the same
    code objects; only the bits of the data differ).  The clock this GPU holds under matrix load depends on the operands, so the
    zero-operand figure is what a kernel's structure allows and the other what the part's power management then leaves of it."""
    from eisen_amd import hip
    BF16 = hip.BF16
    rng = np.random.default_rng(7)
    M = 4096
    wm, wn, nprod, nseg = 2048, 5632, 32, 8
    Cs = [ctx.malloc(wm * wn * 4) for _ in range(nprod)]
    c2, G, U, H = (ctx.malloc(M * cols * 2) for cols in (2048, 5632, 5632, 5632))
    out = dict(unit="TFLOP/s")

    def rate(fn, flop, reps):
        for _ in range(2):
            fn()
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        ctx.sync()
        return round(flop * reps / (time.perf_counter() - t0) / 1e12, 1)

    for label in ("zero_operands", "normal_operands"):
        mk = (lambda shape: np.zeros(shape, np.float32)) if label == "zero_operands" else (lambda shape: hip.round_bf16(rng.standard_normal(shape, dtype=np.float32)))
        x2, x5 = ctx.upload(mk((M, 2048)), BF16), ctx.upload(mk((M, 5632)), BF16)
        w22, w52, wg, wu = (ctx.upload(mk(sh), BF16) for sh in ((2048, 2048), (5632, 2048), (2048, 5632), (2048, 5632)))
        A, B = [[x2] * nseg] * nprod, [[x5] * nseg] * nprod
        out[label] = {
            "gemm_tn_bf16_f32out_256x256x32_window, 32 x [2048 x 5632] over 8 x 4096 rows":
                rate(lambda: ctx.gemm_grouped_ksegments(A, B, Cs, [wm] * nprod, [wn] * nprod, M, 0), 2.0 * wm * wn * M * nseg * nprod, 2),
            "gemm_nn_bf16_bf16out_256x128x64, 4096 x 2048 x 5632": rate(lambda: ctx.gemm(x5, w52, c2, BF16, BF16, 0, 0, M, 2048, 5632), 2.0 * M * 2048 * 5632, 30),
            "gemm_nt_bf16_bf16out_256x128x64, 4096 x 2048 x 2048": rate(lambda: ctx.gemm(x2, w22, c2, BF16, BF16, 0, 1, M, 2048, 2048), 2.0 * M * 2048 * 2048, 30),
            "gemm_nn_bf16_swiglu_fwd, 4096 x (5632 + 5632) x 2048": rate(lambda: ctx.gemm_swiglu_forward(x2, wg, wu, G, U, H, BF16, M, 5632, 2048), 4.0 * M * 5632 * 2048, 20),
        }
        for b in (x2, x5, w22, w52, wg, wu):
            b.free()
    for b in Cs + [c2, G, U, H]:
        b.free()
    return out


def pick_dominant(prof, workload):
    sym = by_symbol(prof)
    name = max(sym, key=lambda k: sym[k]["ms"])
    r = roofline_of(name, sym[name], workload, strict=True)
    if len(sym[name]["families"]) > 1:
        r["families"] = sorted(sym[name]["families"])
    return r


def kernel_table(prof):
    rows = []
    for name, e in sorted(prof.items(), key=lambda kv: -kv[1]["ms"]):
        rate = e["work"] / (e["ms"] * 1e-3) if e["ms"] > 0 else 0.0
        flop = e["unit"] == "flop"
        rows.append(dict(kernel=name, ms=round(e["ms"], 3), launches=e["launches"], avg_us=round(1e3 * e["ms"] / e["launches"], 2),
                         rate=round(rate / (1e12 if flop else 1e9), 2), rate_unit="TFLOP/s" if flop else "GB/s",
                         frac=round(rate / (1e12 * PEAK_BF16_TFLOPS if flop else 1e9 * PEAK_HBM_GBS), 4)))
    return rows


# ---------------------------------------------------------------------------------------------
# CPU baseline: the oracle (port of the reference's CPU arms) on a bounded sample
# ---------------------------------------------------------------------------------------------

def cpu_threads():
    return max(1, min(16, os.cpu_count() or 1))


def cpu_baseline_lm(c, seq, mb=1):
    """One micro-step (forward, cross entropy, backward) of a 0-layer and a 1-layer model of the configuration's width
    and vocabulary on mb x seq tokens: the difference is one transformer layer (attention with its S^2 part at this
    seq), the 0-layer run is embedding + final norm + lm_head + cross entropy.  Extrapolated to the full depth."""
    from oracle import cpu_ref as R
    threads = cpu_threads()
    R.set_threads(threads)
    times = {}
    for layers in (0, 1):
        cfg = dict(arch(c), layers=layers)
        g = R.Graph()
        lm = R.TransformerLM(g, **cfg)
        for pid, (_, w) in enumerate(gen.lm_weights(5, **cfg)):
            g.load_tensor_data(pid, w)
        g.mark_params()
        x, y = gen.lm_batch(9, mb, seq, c["vocab"], "zipf")
        t0 = time.perf_counter()
        lm.micro_step(x, y)
        times[layers] = time.perf_counter() - t0
        del lm, g
    per_layer = max(times[1] - times[0], 1e-9)
    per_token = (c["layers"] * per_layer + times[0]) / (mb * seq)
    note = "" if seq >= c["seq"] else f" (at seq {seq} the S^2 attention term has {seq / c['seq']:.2g} of its share at seq {c['seq']})"
    return dict(value=round(1.0 / per_token, 3), unit="tokens/s", cores=threads, kind="port",
                sample=(f"oracle forward + cross entropy + backward on {mb} x {seq} tokens of this width and vocabulary: 0 layers "
                        f"(embedding, final norm, lm_head, CE) {times[0]:.1f} s, 1 layer {times[1]:.1f} s, extrapolated to {c['layers']} layers{note}; "
                        f"AdamW excluded; the reference's CPU path itself is single-threaded, the port runs its row loops on {threads} threads "
                        f"with identical results"))


# ---------------------------------------------------------------------------------------------
# workloads
# ---------------------------------------------------------------------------------------------

def bench_lm(name, steps, warmup, with_cpu=True, recompute=False, window=True, beside=True, meet_us=None):
    from eisen_amd import graph as G
    from eisen_amd import hip
    c = CONFIGS[name]
    ctx = hip.Context(0)
    if meet_us is not None:   # A/B of the windowed weight-gradient GEMM's meeting points (library default: 40 us; 0 = none)
        ctx.gemm_window_meet(meet_us)
    g = G.Graph(ctx, G.BF16_MIXED)
    lm = G.TransformerLM(g, **arch(c))
    rng = np.random.default_rng(1234)
    for pid in range(g.num_tensors()):
        shape = g.shape(pid)
        if len(shape) == 2:   # matrices N(0, 0.02); norm gains stay 1.0
            g.load_tensor_data(pid, rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02))
    g.mark_params()
    lm.set_checkpointing(recompute)   # per-block recompute: off in the headline run (the reference's train_llm.rs does not use it)
    # weight gradients over the whole accumulation window in one contraction (Graph::set_weight_gradient_window): the sums
    # of train_llm.rs:386-477's micro-batch loop, each gradient read and written once per optimizer step
    win_passes = c["accum"] if window and 2 <= c["accum"] <= 8 else 0
    g.set_weight_gradient_window(win_passes)
    g.set_weight_gradients_beside(beside)   # the library's default; off = every GEMM in tape order on the one stream
    opt = G.AdamW(g, lm.params(), 1e-3)
    opt.config(1e-3, 0.9, 0.95, 1e-8, 0.1, 1.0)      # train_llm.rs:266-270 + grad clip 1.0
    opt.init_moments()
    n_batches = (steps + warmup + 1) * c["accum"]
    batches = [gen.lm_batch(100 + i, c["mb"], c["seq"], c["vocab"], "zipf") for i in range(n_batches)]
    batches = [(x.astype(np.float32), y) for x, y in batches]
    it = iter(batches)

    step_no = [0]

    def one_step():
        # linear warm-up of the reference's CosineScheduler (src/nn/scheduler.rs:45-55; train_llm.rs:391-392)
        opt.config(g.cosine_lr(3e-4, 3e-5, 100, 10000, step_no[0]), 0.9, 0.95, 1e-8, 0.1, 1.0)
        step_no[0] += 1
        opt.zero_grad()
        loss = None
        for _ in range(c["accum"]):
            x, y = next(it)
            loss = lm.micro_step(x, y, want_loss=True)    # train_llm.rs:450 reads every micro-batch's loss
        opt.step()
        return loss

    for _ in range(warmup):
        one_step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    ctx.sync()
    elapsed = time.perf_counter() - t0
    # one more, instrumented step for the per-kernel numbers (not part of `value`)
    ctx.profile_start()
    last_loss = one_step()
    prof = ctx.profile_stop()
    tokens_per_step = c["accum"] * c["mb"] * c["seq"]
    value = steps * tokens_per_step / elapsed
    step_flops = flops_per_token(c) * tokens_per_step
    out = dict(metric="train tokens/sec (fwd+bwd+AdamW)", value=round(value, 1), unit="tokens/s", n_gpus=1, steps=steps, warmup=warmup,
               ms_per_step=round(1e3 * elapsed / steps, 3), higher_is_better=True, scaling="weak", vs_baseline=None, dtype="bf16",
               data="synthetic",
               config=dict(workload=c["label"] + (", per-block recompute" if recompute else ""), tokens_per_step=tokens_per_step, parallelism="single GPU",
                           weight_gradient_window=win_passes, weight_gradients_beside=bool(beside), recompute=bool(recompute),
                           step_model_tflops=round(step_flops / 1e12, 4),
                           mfma_frac_of_step=round(step_flops / (elapsed / steps) / 1e12 / PEAK_BF16_TFLOPS, 4), last_loss=round(float(last_loss), 4)),
               roofline=pick_dominant(prof, name), kernels=kernel_table(prof))
    out["roofline"]["mfma_ceiling"] = mfma_ceiling(ctx)
    if name == "c5" and win_passes and PROBES:
        out["roofline"]["gemms_alone_by_operand_data"] = gemms_by_operand_data(ctx)
    ctx.close()
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline_lm(c, c["seq"], 1 if name == "c5" else 8)
    return out


def bench_c3(steps, warmup, hd=64):
    """Config 3: causal GQA flash attention forward + backward, B8 S1024 Hq16 Hkv4 hd64 bf16, layout [B,H,S,hd].
    hd = 128 (--head-dim 128) keeps the tokens, the model width (Hq * hd = 1024) and so the algorithmic flops, with 8 query and
    2 KV heads: the same problem at the head size where a score tile costs half the softmax work per MFMA."""
    from eisen_amd import hip
    from oracle import cpu_ref as R
    B, S = 8, 1024
    Hq, Hkv = 1024 // hd, 256 // hd
    ctx = hip.Context(0)
    sd = 1.0 / 8
    scale = float(1.0 / np.sqrt(hd))     # 1/8 at config 3's head size
    q, do = gen.normal(600, (B, Hq, S, hd), sd), gen.normal(601, (B, Hq, S, hd), sd)
    k, v = gen.normal(602, (B, Hkv, S, hd), sd), gen.normal(603, (B, Hkv, S, hd), sd)
    dq_, dk_, dv_, ddo = (ctx.upload(t, hip.BF16) for t in (q, k, v, do))
    out, lse = ctx.malloc(q.size * 2), ctx.malloc(B * Hq * S * 4)
    gq, gk, gv = ctx.malloc(q.size * 2), ctx.malloc(k.size * 2), ctx.malloc(k.size * 2)
    qs, ks = (Hq * S * hd, hd, S * hd), (Hkv * S * hd, hd, S * hd)

    def step():
        ctx.attention_forward(dq_, dk_, dv_, out, lse, hip.BF16, B, S, Hq, Hkv, hd, scale, True, qs, ks)
        ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, hip.BF16, B, S, Hq, Hkv, hd, scale, True, qs, ks)

    for _ in range(warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    elapsed = time.perf_counter() - t0
    ctx.profile_start()
    for _ in range(steps):
        step()
    prof = ctx.profile_stop()
    bwd_keys = [k_ for k_ in prof if k_.startswith("attn_bwd")]
    bwd_ms_events_each = sum(prof[k_]["ms"] for k_ in bwd_keys) / steps   # one pair of events around every launch: adds a few us to a 50 us kernel
    # the backward's duration: one pair of events around `steps` backward calls in a row (2 * steps launches on the stream)
    ctx.timer_start()
    for _ in range(steps):
        ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, hip.BF16, B, S, Hq, Hkv, hd, scale, True, qs, ks)
    bwd_ms = ctx.timer_stop() / steps
    bwd_flops = 4 * 2 * hd * (S * (S + 1) / 2) * B * Hq          # 34.39 GFLOP: four GEMMs, causal pairs, no recompute
    achieved = bwd_flops / (bwd_ms * 1e-3) / 1e12
    tokens = B * S
    ceiling = mfma_ceiling(ctx)
    ctx.close()
    # CPU: the unfused chain on one batch element and one KV group (4 query heads), scaled by B*Hkv
    R.set_threads(1)
    t1 = time.perf_counter()
    grp = Hq // Hkv
    R.attention_chain(np.ascontiguousarray(q[:1, :grp].transpose(0, 2, 1, 3)), np.ascontiguousarray(k[:1, :1].transpose(0, 2, 1, 3)),
                       np.ascontiguousarray(v[:1, :1].transpose(0, 2, 1, 3)), np.ascontiguousarray(do[:1, :grp].transpose(0, 2, 1, 3)), np.float32(scale))
    cpu_s = (time.perf_counter() - t1) * B * Hkv
    return dict(metric="flash-attention fwd+bwd tokens/sec (config 3)", value=round(steps * tokens / elapsed, 1), unit="tokens/s", n_gpus=1,
                steps=steps, warmup=warmup, ms_per_step=round(1e3 * elapsed / steps, 4), higher_is_better=True, scaling="weak",
                vs_baseline=None, dtype="bf16", data="synthetic",
                config=dict(workload=f"config3 causal GQA flash attention fwd+bwd, B8 S1024 Hq{Hq} Hkv{Hkv} hd{hd}, [B,H,S,hd]" +
                            ("" if hd == 64 else " (config 3's tokens and width at another head size)")),
                roofline=dict(bound="mfma", achieved=round(achieved, 2), peak=PEAK_BF16_TFLOPS, unit="TFLOP/s",
                              frac=round(achieved / PEAK_BF16_TFLOPS, 4), traffic=MEASURED_TRAFFIC["c3"]["attn_bwd"] if hd == 64 else None,
                              traffic_source=TRAFFIC_SOURCE["c3"] if hd == 64 else None,
                              kernel="attn_bwd (" + " + ".join(sorted(bwd_keys)) + ")", bwd_us=round(1e3 * bwd_ms, 2),
                              timing=f"HIP events around {steps} backward calls in a row; with a pair of events around every launch of the fwd+bwd steps "
                                     f"the two kernels sum to {round(1e3 * bwd_ms_events_each, 2)} us",
                              algorithmic_gflop=round(bwd_flops / 1e9, 2), mfma_ceiling=ceiling),
                kernels=kernel_table(prof),
                cpu_baseline=dict(value=round(tokens / cpu_s, 2), unit="tokens/s", cores=1, kind="port",
                                  sample="oracle unfused attention chain fwd+bwd on 1 of 32 (batch, KV group) slices, scaled x32"))


def bench_c3_ablation(steps, warmup):
    """Where the time of the two config-3 backward kernels goes: each run leaves one part of their tile loop out
    (eisen_hip_attention_ablation; results wrong by construction, memory accesses unchanged) and reports the kernels' average
    durations; what a run gains against the full kernels is that part's share of the critical path."""
    from eisen_amd import hip
    B, S, Hq, Hkv, hd = 8, 1024, 16, 4, 64
    ctx = hip.Context(0)
    q, do = gen.normal(600, (B, Hq, S, hd), 1.0 / 8), gen.normal(601, (B, Hq, S, hd), 1.0 / 8)
    k, v = gen.normal(602, (B, Hkv, S, hd), 1.0 / 8), gen.normal(603, (B, Hkv, S, hd), 1.0 / 8)
    dq_, dk_, dv_, ddo = (ctx.upload(t, hip.BF16) for t in (q, k, v, do))
    out, lse = ctx.malloc(q.size * 2), ctx.malloc(B * Hq * S * 4)
    gq, gk, gv = ctx.malloc(q.size * 2), ctx.malloc(k.size * 2), ctx.malloc(k.size * 2)
    qs, ks = (Hq * S * hd, hd, S * hd), (Hkv * S * hd, hd, S * hd)
    ctx.attention_forward(dq_, dk_, dv_, out, lse, hip.BF16, B, S, Hq, Hkv, hd, 0.125, True, qs, ks)
    parts = ["none (the kernels as shipped)", "LDS transpose reads", "16-byte LDS operand reads", "MFMAs after the softmax", "global-to-LDS tile loads",
             "softmax arithmetic", "S and dP MFMAs", "none (again, after the others)"]
    rows = []
    for i, label in enumerate(parts):
        ctx.attention_ablation(i % 7)
        for _ in range(warmup):
            ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, hip.BF16, B, S, Hq, Hkv, hd, 0.125, True, qs, ks)
        ctx.sync()
        ctx.profile_start()
        for _ in range(steps):
            ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, hip.BF16, B, S, Hq, Hkv, hd, 0.125, True, qs, ks)
        prof = ctx.profile_stop()
        rows.append(dict(left_out=label, dq_us=round(1e3 * prof["attn_bwd_dq_bf16"]["ms"] / steps, 2), dkv_us=round(1e3 * prof["attn_bwd_dkv_bf16"]["ms"] / steps, 2)))
    ctx.attention_ablation(0)
    ctx.close()
    return dict(metric="config-3 attention backward kernel durations with one part of the tile loop left out", unit="us", steps=steps, warmup=warmup,
                config=dict(workload="config3 causal GQA flash attention backward, B8 S1024 Hq16 Hkv4 hd64, [B,H,S,hd]"), rows=rows)


def bench_c2(steps, warmup):
    """Config 2: fused softmax-cross-entropy forward+backward, bf16 [8192 x 32000]."""
    from eisen_amd import hip
    from oracle import cpu_ref as R
    rows, V = 8192, 32000
    ctx = hip.Context(0)
    rng = np.random.default_rng(7)
    x = rng.standard_normal((rows, V), dtype=np.float32) * np.float32(2.0)
    t = rng.integers(0, V, rows)
    dx, dt = ctx.upload(x, hip.BF16), ctx.upload(t.astype(np.int32))
    dl, rl, lo = ctx.malloc(rows * V * 2), ctx.malloc(rows * 4), ctx.malloc(4)

    def step():
        ctx.cross_entropy(dx, dt, dl, rl, lo, hip.BF16, rows, V, 1.0 / rows)

    for _ in range(warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    elapsed = time.perf_counter() - t0
    ctx.profile_start()
    for _ in range(steps):
        step()
    prof = ctx.profile_stop()
    roofline = pick_dominant(prof, "c2")
    # What a plain copy of the same bytes (logits read, gradient written) reaches on this GPU, in this run: the practical
    # ceiling of a kernel that streams 524 MB in and 524 MB out, next to the published 8 TB/s the fraction is quoted against.
    for _ in range(warmup):
        ctx.cast(dx, hip.BF16, dl, hip.BF16, rows * V)
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        ctx.cast(dx, hip.BF16, dl, hip.BF16, rows * V)
    ctx.sync()
    copy_gbs = steps * 2.0 * rows * V * 2 / (time.perf_counter() - t0) / 1e9
    roofline["copy_of_same_bytes"] = dict(achieved=round(copy_gbs, 1), unit="GB/s", frac=round(copy_gbs / 8000.0, 4))
    ctx.close()
    R.set_threads(1)
    sample = 64
    xs = hip.round_bf16(x[:sample])
    t1 = time.perf_counter()
    R.cross_entropy(xs, t[:sample])
    cpu_rows_s = sample / (time.perf_counter() - t1)
    return dict(metric="fused softmax-cross-entropy fwd+bwd rows/sec (config 2)", value=round(steps * rows / elapsed, 1), unit="rows/s", n_gpus=1,
                steps=steps, warmup=warmup, ms_per_step=round(1e3 * elapsed / steps, 4), higher_is_better=True, scaling="weak", vs_baseline=None,
                dtype="bf16", data="synthetic", config=dict(workload="config2 fused softmax-CE fwd+bwd, bf16 logits [8192 x 32000]"),
                roofline=roofline, kernels=kernel_table(prof),
                cpu_baseline=dict(value=round(cpu_rows_s, 2), unit="rows/s", cores=1, kind="port", sample=f"oracle CE fwd+bwd on {sample} of 8192 rows"))


def brief(r):
    """The part of a workload's line that the combined line keeps."""
    keep = ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "config", "roofline", "cpu_baseline")
    return {k: r[k] for k in keep if k in r}


def bench_c3_timeline(steps, warmup):
    """Where a wave of the three config-3 attention kernels spends its life: the kernels drop time stamps of every wave's progress
    (eisen_hip_attention_timeline, the GPU's 100 MHz counter and its shader clock; the results are the usual ones) and this
    reports, per kernel and in microseconds, the phases between the stamps averaged over the waves, the span from the first wave's
    entry to the last wave's end and how far apart the waves finish."""
    from eisen_amd import hip
    B, S, Hq, Hkv, hd = 8, 1024, 16, 4, 64
    ctx = hip.Context(0)
    q, do = gen.normal(600, (B, Hq, S, hd), 1.0 / 8), gen.normal(601, (B, Hq, S, hd), 1.0 / 8)
    k, v = gen.normal(602, (B, Hkv, S, hd), 1.0 / 8), gen.normal(603, (B, Hkv, S, hd), 1.0 / 8)
    dq_, dk_, dv_, ddo = (ctx.upload(t, hip.BF16) for t in (q, k, v, do))
    out, lse = ctx.malloc(q.size * 2), ctx.malloc(B * Hq * S * 4)
    gq, gk, gv = ctx.malloc(q.size * 2), ctx.malloc(k.size * 2), ctx.malloc(k.size * 2)
    qs, ks = (Hq * S * hd, hd, S * hd), (Hkv * S * hd, hd, S * hd)
    waves = 4096                      # the forward runs 1024 blocks of four waves, the backward kernels 512
    stamps = ctx.malloc(3 * waves * 16 * 8, zero=True)
    ctx.attention_timeline(stamps, waves)
    acc = None
    for i in range(warmup + steps):
        ctx.memset_zero(stamps, 3 * waves * 16 * 8)
        ctx.attention_forward(dq_, dk_, dv_, out, lse, hip.BF16, B, S, Hq, Hkv, hd, 0.125, True, qs, ks)
        ctx.attention_backward(dq_, dk_, dv_, out, ddo, lse, gq, gk, gv, hip.BF16, B, S, Hq, Hkv, hd, 0.125, True, qs, ks)
        ctx.sync()
        if i < warmup:
            continue
        t = ctx.download(stamps, (3, waves, 8, 2), np.int64).astype(np.float64)
        rows = []
        for kern in range(3):
            w = t[kern, :, :, 0] * 1e-2          # microseconds (100 MHz)
            cyc = t[kern, :, :, 1]
            live = w[:, 0] > 0
            w, cyc = w[live], cyc[live]
            t0 = w[:, 0].min()
            second = w[:, 6] > 0                 # waves with a second block
            end = np.where(second, w[:, 6], w[:, 3])
            loop = (w[:, 2] - w[:, 1]) + np.where(second, w[:, 5] - w[:, 4], 0.0)
            loop_cyc = (cyc[:, 2] - cyc[:, 1]) + np.where(second, cyc[:, 5] - cyc[:, 4], 0.0)
            rows.append([float(live.sum()), float((w[:, 1] - w[:, 0]).mean()), float(loop.mean()), float((w[:, 3] - w[:, 2]).mean()),
                         float(np.where(second, w[:, 4] - w[:, 3], 0.0).sum() / max(1, second.sum())),
                         float(np.where(second, w[:, 6] - w[:, 5], 0.0).sum() / max(1, second.sum())),
                         float(end.max() - t0), float(np.median(end) - t0), float(end.min() - t0), float(loop_cyc.sum() / (loop.sum() * 1e3))])
        acc = np.array(rows) if acc is None else acc + np.array(rows)
    acc /= steps
    ctx.attention_timeline(None, 0)
    # the dK/dV kernel's tile loop rebuilt from the same instructions on made-up data: what each part costs alone and together
    model = {}
    for label, parts in (("mfma", 1), ("mfma_valu", 3), ("mfma_valu_lds", 7), ("tile_loads", 8), ("all", 15)):
        for wps in (1, 2):
            model[f"{label}_{wps}_per_simd"] = round(ctx.attention_tile_model(parts, wps, 4000), 1)
    # the tile loop of a one-pass backward (S and dP once, dQ partials per 128-key chunk), and the two kernels it would need around it
    onepass = {}
    for label, parts in (("tile_with_partial_stores", 16), ("tile_without_partial_stores", 32)):
        onepass[f"{label}_ns_per_tile_and_simd"] = round(ctx.attention_tile_model(parts, 2, 4000), 1)
    for chunk in (128, 256):
        d_us, sum_us = ctx.attention_onepass_parts(8 * 16 * 1024, 1024, chunk)
        onepass["rowdot_prepass_us"] = round(d_us, 2)
        onepass[f"partial_sum_chunk{chunk}_us"] = round(sum_us, 2)
    ctx.close()
    names = ["attn_fwd_bf16", "attn_bwd_dq_bf16", "attn_bwd_dkv_bf16"]
    keys = ["waves", "entry_to_first_loop_us", "tile_loops_us", "first_block_stored_us", "to_second_loop_us", "second_block_stored_us",
            "first_entry_to_last_end_us", "first_entry_to_median_end_us", "first_entry_to_first_end_us", "loop_clock_ghz"]
    return dict(metric="config-3 attention kernels: a wave's life by phase (in-kernel time stamps, mean over waves)", unit="us", steps=steps, warmup=warmup,
                config=dict(workload="config3 causal GQA flash attention fwd+bwd, B8 S1024 Hq16 Hkv4 hd64, [B,H,S,hd]"),
                rows=[dict(kernel=n, **{k_: round(float(x), 2) for k_, x in zip(keys, r)}) for n, r in zip(names, acc)],
                dkv_tile_loop_model_ns_per_tile_and_simd=model, one_pass_model=onepass)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="all", choices=["all", "c5", "c4", "c3", "c2"])
    ap.add_argument("--head-dim", type=int, default=64, choices=[32, 64, 128], help="c3: head size (the token count and Hq * hd = 1024 stay)")
    ap.add_argument("--ablation", action="store_true", help="c3: time the backward kernels with one part of their tile loop left out at a time")
    ap.add_argument("--timeline", action="store_true", help="c3: where a wave of the three kernels spends its life (time stamps dropped inside the kernels)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg (profiling runs)")
    ap.add_argument("--no-probes", action="store_true", help="skip the launches that only measure the GPU (roofline.mfma_ceiling, roofline.gemms_alone_by_operand_data): "
                    "for kernel traces, whose per-kernel averages they would enter")
    ap.add_argument("--no-window", action="store_true", help="c5: form every micro-batch's weight gradients in its own backward pass, as the reference does, "
                    "instead of once per optimizer step over the whole accumulation window")
    ap.add_argument("--window-meet-us", type=int, default=None, help="c5: longest wait at the meeting points of the windowed weight-gradient GEMM "
                    "(library default 40; 0 switches them off)")
    ap.add_argument("--no-beside", action="store_true", help="c4: keep the weight-gradient GEMMs of narrow layers on the main stream, in tape order")
    ap.add_argument("--recompute", action="store_true", help="c5 / c4: per-block recompute (lower activation memory, one more forward pass per block)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    global PROBES
    PROBES = not args.no_probes
    w = args.workload
    if w in ("all", "c5"):
        out = bench_lm("c5", args.steps if args.steps is not None else 3, args.warmup if args.warmup is not None else 1, not args.no_cpu, args.recompute, not args.no_window, not args.no_beside, args.window_meet_us)
        if w == "all":
            out["other_configs"] = dict(c4=brief(bench_lm("c4", 20, 3, not args.no_cpu)), c3=brief(bench_c3(20, 3)), c2=brief(bench_c2(20, 3)))
            if not args.no_window:   # the same step in the reference's accumulation order: every pass forms and adds its own dW
                ref_order = brief(bench_lm("c5", 3, 1, False, args.recompute, False, not args.no_beside))
                out["other_configs"]["c5_per_pass_weight_gradients"] = {k: ref_order[k] for k in ("value", "unit", "ms_per_step", "steps", "warmup", "config")}
    elif w == "c4":
        out = bench_lm("c4", args.steps if args.steps is not None else 20, args.warmup if args.warmup is not None else 3, not args.no_cpu, args.recompute, not args.no_window, not args.no_beside)
    elif w == "c3" and args.ablation:
        out = bench_c3_ablation(args.steps or 20, args.warmup if args.warmup is not None else 3)
    elif w == "c3" and args.timeline:
        out = bench_c3_timeline(args.steps or 10, args.warmup if args.warmup is not None else 3)
    elif w == "c3":
        out = bench_c3(args.steps or 20, args.warmup if args.warmup is not None else 3, args.head_dim)
    else:
        out = bench_c2(args.steps or 20, args.warmup if args.warmup is not None else 3)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
