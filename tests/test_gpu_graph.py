"""GPU tests of the host Graph / nn / AdamW layer through include/eisen_graph.h.

The reference's own GPU tests (tests/gpu_kernels.rs, phase2_*_gpu.rs, test_grad_accum.rs) are
replayed against the new Device::Gpu backend, then the composed training step is compared
with the CPU oracle on the same seeded inputs: config 1 in f32 (rtol 1e-4) and a bf16 mixed
step of the config-4 architecture (rtol 2e-2 on gradients).
"""
import numpy as np
import pytest

from eisen_amd import graph as G
from eisen_amd.lib import EisenHipError
from oracle import cpu_ref as R
from tests import gen
from tests.gpu_util import assert_close, ctx  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.fixture
def g(ctx):
    gr = G.Graph(ctx, G.FP32)
    yield gr
    gr.close()


# ---- the reference's per-op GPU tests -------------------------------------------------------

def test_add_mul_matmul_reference_vectors(g):
    # tests/gpu_kernels.rs:27-41, :52-67, :79-103
    a, b = g.alloc((2, 2), [1, 2, 3, 4]), g.alloc((2, 2), [0.5, 1.5, 2.5, 3.5])
    c = g.add(a, b)
    assert g.sync_to_cpu(c).reshape(-1).tolist() == [1.5, 3.5, 5.5, 7.5]
    g.backward(c)
    assert g.sync_grad_to_cpu(a).reshape(-1).tolist() == [1.0] * 4 and g.sync_grad_to_cpu(b).reshape(-1).tolist() == [1.0] * 4
    a, b = g.alloc((3,), [2, -3, 4]), g.alloc((3,), [5, 2, -1])
    c = g.mul(a, b)
    assert g.sync_to_cpu(c).tolist() == [10.0, -6.0, -4.0]
    g.backward(c)
    assert g.sync_grad_to_cpu(a).tolist() == [5.0, 2.0, -1.0] and g.sync_grad_to_cpu(b).tolist() == [2.0, -3.0, 4.0]
    a, b = g.alloc((2, 3), [1, 2, 3, 4, 5, 6]), g.alloc((3, 2), [7, 8, 9, 1, 2, 3])
    c = g.matmul(a, b)
    assert g.sync_to_cpu(c).reshape(-1).tolist() == [31.0, 19.0, 85.0, 55.0]
    g.backward(c)
    assert g.sync_grad_to_cpu(a).reshape(-1).tolist() == [15.0, 10.0, 5.0, 15.0, 10.0, 5.0]
    assert g.sync_grad_to_cpu(b).reshape(-1).tolist() == [5.0, 5.0, 7.0, 7.0, 9.0, 9.0]


def test_broadcast_add_reference(g):
    # tests/phase1.rs:8-20 (the [1,3] row broadcast onto [2,3]); grads through a broadcast
    a, b = g.alloc((2, 3), [1, 2, 3, 4, 5, 6]), g.alloc((1, 3), [10, 20, 30])
    c = g.add(a, b)
    assert g.sync_to_cpu(c).reshape(-1).tolist() == [11, 22, 33, 14, 25, 36]
    g.backward(c)
    assert g.sync_grad_to_cpu(a).reshape(-1).tolist() == [1.0] * 6
    assert g.sync_grad_to_cpu(b).reshape(-1).tolist() == [2.0] * 3


def test_silu_gather_rmsnorm_ce_rope_reference(g):
    # SiLU closed form, tests/gpu_kernels.rs:114-152
    x = np.array([-2.0, -1.0, 0.0, 1.0, 2.0], np.float32)
    a = g.alloc((5,), x)
    s = g.silu(a)
    sig = 1 / (1 + np.exp(-x.astype(np.float64)))
    assert np.abs(g.sync_to_cpu(s) - x * sig).max() < 1e-5
    g.backward(s)
    assert np.abs(g.sync_grad_to_cpu(a) - sig * (1 + x * (1 - sig))).max() < 1e-5
    # gather with a collision, tests/gpu_kernels.rs:164-206; indices are an f32 tensor
    w = g.alloc((3, 2), [0.1, 0.2, 0.3, 0.4, 0.5, 0.6])
    idx = g.alloc((4,), [2.0, 0.0, 2.0, 1.0])
    c = g.gather(w, idx)
    assert np.abs(g.sync_to_cpu(c).reshape(-1) - [0.5, 0.6, 0.1, 0.2, 0.5, 0.6, 0.3, 0.4]).max() < 1e-5
    g.backward(c)
    assert g.sync_grad_to_cpu(w).reshape(-1).tolist() == [1, 1, 1, 1, 2, 2]
    # rmsnorm smoke, tests/gpu_kernels.rs:209-259 (+ values against the oracle)
    xd = np.array([[1, -2, 3, -4], [0.1, 0.2, -0.1, 0.0]], np.float32)
    xi, wi = g.alloc((2, 4), xd), g.alloc((4,), np.ones(4))
    o = g.rms_norm(xi, wi, 1e-5)
    eo, er = R.rms_norm_fwd(xd, np.ones(4, np.float32), 1e-5)
    assert_close(g.sync_to_cpu(o), eo, 1e-4, "rms")
    g.backward(o)
    egx, egw = R.rms_norm_bwd(xd, np.ones(4, np.float32), er, np.ones((2, 4), np.float32))
    assert_close(g.sync_grad_to_cpu(xi), egx, 1e-4, "rms dx")
    assert_close(g.sync_grad_to_cpu(wi), egw, 1e-4, "rms dw")
    # cross entropy, tests/gpu_kernels.rs:262-289
    lg = g.alloc((2, 3), [2.0, 1.0, 0.1, 0.0, 3.0, 0.5])
    loss = g.cross_entropy(lg, [0, 1])
    assert abs(g.sync_to_cpu(loss).reshape(-1)[0] - 0.27) < 0.05
    g.backward(loss)
    gr = g.sync_grad_to_cpu(lg).reshape(-1)
    assert gr[0] < 0 < gr[1] and gr[2] > 0 and gr[3] > 0 and gr[4] < 0 < gr[5]
    with pytest.raises(EisenHipError):
        g.cross_entropy(lg, [0, 3])                      # target out of range: an error, as the reference panics
    # rope, tests/gpu_kernels.rs:485-513
    q = g.alloc((1, 2, 4), np.ones(8))
    r = g.rope(q, 4)
    rd = g.sync_to_cpu(r).reshape(-1)
    assert rd[:4].tolist() == [1.0] * 4 and abs(rd[4] - (0.5403 - 0.8414)) < 1e-3 and abs(rd[5] - (0.5403 + 0.8414)) < 1e-3
    g.backward(r)
    qg = g.sync_grad_to_cpu(q).reshape(-1)
    assert abs(qg[4] - (0.5403 + 0.8414)) < 1e-3 and abs(qg[5] - (0.5403 - 0.8414)) < 1e-3


def test_bmm_softmax_flash_reference(g):
    # tests/gpu_kernels.rs:344-376
    q = g.alloc((2, 2, 3), [1, 0, 1, 0, 1, 0, 1, 1, 1, 0, 0, 1])
    k = g.alloc((2, 2, 3), [1, 0, 1, 0, 1, 0, 1, 0, 0, 0, 0, 1])
    s = g.bmm(q, k, True)
    assert g.sync_to_cpu(s).reshape(-1)[:4].tolist() == [2.0, 0.0, 0.0, 1.0]
    p = g.softmax(s)
    pv = g.sync_to_cpu(p).reshape(-1)
    assert abs(pv[0] - 0.88079) < 1e-4 and abs(pv[1] - 0.11920) < 1e-4
    g.backward(p)
    assert np.any(g.sync_grad_to_cpu(q) != 0) and np.any(g.sync_grad_to_cpu(k) != 0)
    # flash == materialised chain, tests/gpu_kernels.rs:403-429
    qd = [1, 0, 1, 0, 0, 1, 0, 1, 1, 1, 0, 0]
    vd = [0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.1, 1.2]
    q, k, v = g.alloc((1, 3, 4), qd), g.alloc((1, 3, 4), qd), g.alloc((1, 3, 4), vd)
    sc = g.mul(g.bmm(q, k, True), g.alloc((1, 3, 3), np.full(9, 0.5)))
    ref = g.sync_to_cpu(g.bmm(g.softmax(sc), v, False))
    g.set_no_grad(True)
    fl = g.sync_to_cpu(g.flash_attention(q, k, v, 0.5, False))
    g.set_no_grad(False)
    assert np.abs(fl - ref).max() < 1e-4


def test_gradient_checkpoint_primitives_are_deterministic(g):
    # tests/gpu_kernels.rs:560-610: a no_grad forward equals the recomputed forward bit for bit
    lm = G.TransformerLM(g, 64, 32, 4, 2, 64, 1, False)
    g.mark_params()
    x, _ = gen.lm_batch(70, 2, 16, 64)
    g.set_no_grad(True)
    sp = g.mark_save_point()
    first = g.sync_to_cpu(lm.forward(g.input(x)))
    g.restore_save_point(sp)
    assert g.num_tensors() == sp and g.tape_len() == 0
    g.set_no_grad(False)
    second = g.sync_to_cpu(lm.forward(g.input(x)))
    assert np.array_equal(first, second) and g.tape_len() > 0
    g.clear_activations()
    assert g.num_tensors() == g.num_params() and g.tape_len() == 0


def test_restore_save_point_keep_moves_one_tensor_down(g):
    a = g.alloc((2, 2), [1, 2, 3, 4])
    g.mark_params()
    sp = g.mark_save_point()
    g.set_no_grad(True)
    b = g.add(a, a)
    c = g.mul(b, b)
    d = g.add(c, a)
    kept = g.restore_save_point_keep(sp, c)
    g.set_no_grad(False)
    assert kept == sp and g.num_tensors() == sp + 1 and d >= g.num_tensors()
    assert g.sync_to_cpu(kept).reshape(-1).tolist() == [4.0, 16.0, 36.0, 64.0]
    with pytest.raises(EisenHipError):
        g.restore_save_point_keep(sp + 1, sp)   # the tensor to keep lies below the save point


@pytest.mark.parametrize("precision,fused", [(G.FP32, True), (G.FP32, False), (G.BF16_MIXED, True), (G.BF16_MIXED, False)],
                         ids=["f32-fused", "f32-chain", "bf16-fused", "bf16-chain"])
def test_per_block_recompute_gives_the_same_bits_and_a_lower_high_water_mark(ctx, precision, fused):
    # TransformerLM::set_checkpointing on mark_save_point / restore_save_point (src/graph/mod.rs:332-365): each block's
    # forward re-runs inside backward.  Deterministic kernels => losses and every gradient bit-identical to the plain
    # step, over two accumulated micro-batches; the peak of pool bytes in use drops.
    cfg = dict(vocab=512, hidden=256, heads=4, kv_heads=2, ffn=512, layers=6, tie=False)
    mb, seq = 4, 128
    batches = [gen.lm_batch(900 + i, mb, seq, cfg["vocab"]) for i in range(2)]
    results = []
    for checkpointing in (False, True):
        gg = G.Graph(ctx, precision)
        lm = G.TransformerLM(gg, **cfg)
        for pid, (_, w) in enumerate(gen.lm_weights(33, perturb_norm=0.1, **cfg)):
            gg.load_tensor_data(pid, w)
        gg.mark_params()
        lm.set_fused(fused)
        lm.set_checkpointing(checkpointing)
        params = lm.params()
        opt = G.AdamW(gg, params, 1e-3)
        opt.zero_grad()
        ctx.sync()
        ctx.pool_peak(reset=True)
        base = ctx.pool_stats()[0]
        losses = [lm.micro_step(x, y) for x, y in batches]
        peak = ctx.pool_peak() - base
        assert gg.num_tensors() == gg.num_params() and gg.tape_len() == 0
        results.append((losses, [gg.sync_grad_to_cpu(p) for p in params], peak))
        gg.close()
    (l0, g0, peak0), (l1, g1, peak1) = results
    assert l0 == l1
    for i, (a, b) in enumerate(zip(g0, g1)):
        assert a.any() and np.array_equal(a, b), f"gradient of parameter {i} differs under per-block recompute"
    assert peak1 < 0.6 * peak0, (peak0, peak1)


@pytest.mark.parametrize("fused,checkpointing", [(True, False), (False, False), (True, True)], ids=["fused", "chain", "fused-recompute"])
def test_weight_gradient_window_sums_over_micro_batches(ctx, fused, checkpointing):
    # Graph::set_weight_gradient_window: the dB += A^T dC of every Linear layer (src/graph/ops/linear.rs:279-287) waits
    # for the end of a window of backward passes and runs as one contraction over all of them.  Against the same passes
    # without a window: losses and every gradient the window does not touch (norm gains, embedding) bit-identical -- the
    # chain of activation gradients must not notice that its buffers are kept -- and the windowed gradients equal up to
    # the rounding order of an f32 sum.  A full window (3 passes, gradients assigned), then a partial one that a gradient
    # read ends (2 passes, gradients added to); nothing stays allocated afterwards.
    cfg = dict(vocab=1024, hidden=1024, heads=8, kv_heads=8, ffn=2048, layers=2, tie=False)
    mb, seq = 2, 128
    batches = [gen.lm_batch(950 + i, mb, seq, cfg["vocab"]) for i in range(5)]
    results = []
    for window in (0, 3):
        gg = G.Graph(ctx, G.BF16_MIXED)
        lm = G.TransformerLM(gg, **cfg)
        names = []
        for pid, (name, w) in enumerate(gen.lm_weights(34, perturb_norm=0.1, **cfg)):
            gg.load_tensor_data(pid, w)
            names.append(name)
        gg.mark_params()
        lm.set_fused(fused)
        lm.set_checkpointing(checkpointing)
        gg.set_weight_gradient_window(window)
        params = lm.params()
        opt = G.AdamW(gg, params, 1e-3)
        opt.zero_grad()
        ctx.sync()
        base = ctx.pool_stats()[0]
        ctx.profile_start()
        losses = [lm.micro_step(x, y) for x, y in batches]
        grads = [gg.sync_grad_to_cpu(p) for p in params]
        prof = ctx.profile_stop()
        assert gg.num_tensors() == gg.num_params() and gg.tape_len() == 0
        ctx.sync()
        assert ctx.pool_stats()[0] == base, "buffers kept for the window were not given back"
        launches = sum(e["launches"] for k, e in prof.items() if k.endswith("_window"))
        assert launches == (2 if window else 0), prof.keys()
        results.append((losses, grads, [names[p] for p in params]))
        gg.close()
    (l0, g0, names), (l1, g1, _) = results
    assert l0 == l1
    windowed = 0
    for name, a, b in zip(names, g0, g1):
        assert a.any(), name
        if a.ndim == 2 and "embed" not in name:
            assert_close(b, a, 1e-4, f"windowed gradient of {name}")
            windowed += 1
        else:
            assert np.array_equal(a, b), f"gradient of {name} differs although the window does not hold it"
    assert windowed == 7 * cfg["layers"] + 1


def test_weight_gradient_window_flushes_when_a_gradient_is_read_cleared_or_outgrows_it(ctx):
    # The corners of Graph::set_weight_gradient_window on a two-matmul graph whose weight is used twice per pass: a
    # gradient read in the middle of a window sees every pass so far; zero_grad in the middle of a window discards what
    # the window held (added, then cleared, as the reference's order of calls would); more passes than the window fit
    # in any number of launches; turning the window off finishes what it holds.  Against the same calls without a window.
    hidden, rows = 1024, 128
    w0 = gen.normal(41, (hidden, hidden), 0.03)
    xs = [gen.normal(42 + i, (rows, hidden)) for i in range(7)]
    tg = [gen.uniform_ids(60 + i, (rows,), hidden) for i in range(7)]

    def run(window):
        g = G.Graph(ctx, G.BF16_MIXED)
        w = g.alloc(w0.shape, w0)
        g.mark_params()
        g.set_weight_gradient_window(window)
        opt = G.AdamW(g, [w], 1e-3)
        opt.zero_grad()
        ctx.sync()
        base = ctx.pool_stats()[0]
        seen = []

        def one_pass(i):
            x = g.input(xs[i])
            loss = g.cross_entropy(g.matmul(g.matmul(x, w), w), tg[i])
            g.backward(loss)
            g.clear_activations()

        one_pass(0)
        seen.append(g.sync_grad_to_cpu(w))            # read after one pass of a window of three
        one_pass(1)
        one_pass(2)
        one_pass(3)                                     # the fourth pass since zero_grad: the window has been through one flush by now
        seen.append(g.sync_grad_to_cpu(w))
        one_pass(4)
        opt.zero_grad()                                 # one pass pending: it must not come back after the clearing
        one_pass(5)
        g.set_weight_gradient_window(0)                 # finishes pass 5
        one_pass(6)                                     # formed by its own backward pass
        seen.append(g.sync_grad_to_cpu(w))
        ctx.sync()
        assert g.num_tensors() == g.num_params() and ctx.pool_stats()[0] == base
        g.close()
        return seen

    plain, windowed = run(0), run(3)
    for i, (a, b) in enumerate(zip(plain, windowed)):
        assert a.any()
        assert_close(b, a, 1e-4, f"weight gradient at read {i}")


def test_weight_used_twice_per_pass_outgrows_its_window_entry_alone(ctx):
    # A weight used twice per pass fills its eight pieces after four passes of a window of eight.  Only that weight's pieces
    # are contracted then; the other weight's pieces and the pass count stay, so the window still ends with the eighth pass:
    # three launches in all (the early one, then one per weight: the first weight's second contraction adds to its gradient,
    # the other's assigns), nothing left allocated, and the sums of the per-pass order.  196 tiles of 256 x 256 per weight: the
    # size from which a window's contraction runs as one launch.
    hidden, rows = 3584, 128
    w1_0, w2_0 = gen.normal(71, (hidden, hidden), 0.03), gen.normal(72, (hidden, hidden), 0.03)
    xs = [gen.normal(80 + i, (rows, hidden)) for i in range(8)]
    tg = [gen.uniform_ids(90 + i, (rows,), hidden) for i in range(8)]

    def run(window):
        g = G.Graph(ctx, G.BF16_MIXED)
        w1, w2 = g.alloc(w1_0.shape, w1_0), g.alloc(w2_0.shape, w2_0)
        g.mark_params()
        g.set_weight_gradient_window(window)
        opt = G.AdamW(g, [w1, w2], 1e-3)
        opt.zero_grad()
        ctx.sync()
        base = ctx.pool_stats()[0]
        ctx.profile_start()
        for i in range(8):
            loss = g.cross_entropy(g.matmul(g.matmul(g.matmul(g.input(xs[i]), w1), w2), w1), tg[i])
            g.backward(loss)
            g.clear_activations()
        prof = ctx.profile_stop()
        launches = sum(e["launches"] for k, e in prof.items() if k.endswith("_window"))
        ctx.sync()
        left = ctx.pool_stats()[0] - base
        grads = g.sync_grad_to_cpu(w1), g.sync_grad_to_cpu(w2)
        g.close()
        return launches, left, grads

    n_plain, left_plain, plain = run(0)
    n_win, left_win, windowed = run(8)
    assert n_plain == 0 and n_win == 3, (n_plain, n_win)
    assert left_win == left_plain, "operands kept for the window were not given back when it ended"
    for a, b, name in zip(plain, windowed, ("w1", "w2")):
        assert a.any()
        assert_close(b, a, 1e-4, f"weight gradient of {name}")


@pytest.mark.parametrize("tie,checkpointing", [(True, False), (False, False), (True, True)], ids=["tied", "untied", "tied-recompute"])
def test_weight_gradients_beside_the_chain_give_the_same_bits(ctx, tie, checkpointing):
    # Graph::set_weight_gradients_beside (the default): the weight-gradient GEMMs of narrow layers run on the side stream
    # while the main stream goes on with the input gradients.  Same kernels on the same operands => every loss and
    # gradient bit-identical to the run that keeps the reference's tape order on one stream (src/graph/mod.rs:670-796),
    # over two accumulated micro-batches; with tied embeddings the lm_head gradient (side stream) and the embedding
    # scatter (main stream) meet in one buffer.  Nothing stays allocated afterwards.
    cfg = dict(vocab=512, hidden=256, heads=4, kv_heads=2, ffn=512, layers=3, tie=tie)
    mb, seq = 4, 128
    batches = [gen.lm_batch(970 + i, mb, seq, cfg["vocab"], "zipf") for i in range(2)]
    results = []
    for beside in (False, True):
        gg = G.Graph(ctx, G.BF16_MIXED)
        lm = G.TransformerLM(gg, **cfg)
        for pid, (_, w) in enumerate(gen.lm_weights(35, perturb_norm=0.1, **cfg)):
            gg.load_tensor_data(pid, w)
        gg.mark_params()
        lm.set_checkpointing(checkpointing)
        gg.set_weight_gradients_beside(beside)
        params = lm.params()
        opt = G.AdamW(gg, params, 1e-3)
        opt.zero_grad()
        ctx.sync()
        base = ctx.pool_stats()[0]
        losses = [lm.micro_step(x, y) for x, y in batches]
        grads = [gg.sync_grad_to_cpu(p) for p in params]
        assert gg.num_tensors() == gg.num_params() and gg.tape_len() == 0
        ctx.sync()
        assert ctx.pool_stats()[0] == base, "buffers kept for the side stream were not given back"
        results.append((losses, grads))
        gg.close()
    (l0, g0), (l1, g1) = results
    assert l0 == l1
    for i, (a, b) in enumerate(zip(g0, g1)):
        assert a.any() and np.array_equal(a, b), f"gradient of parameter {i} differs when the weight gradients run beside the chain"


# ---- composed training step against the oracle ---------------------------------------------------

def _build_pair(ctx, cfg, weights, precision):
    gg = G.Graph(ctx, precision)
    lm = G.TransformerLM(gg, **cfg)
    og = R.Graph()
    olm = R.TransformerLM(og, **cfg)
    for pid, (name, w) in enumerate(weights):
        assert gg.shape(pid) == w.shape == og.shape(pid), name
        gg.load_tensor_data(pid, w)
        og.load_tensor_data(pid, w)
    gg.mark_params()
    og.mark_params()
    assert lm.params() == olm.params()
    return gg, lm, og, olm


def _train_steps(ctx, cfg, precision, mb, seq, steps, accum, rtol_grad, seed=1, fused=True, dist="uniform", clip=0.0, perturb_norm=0.05,
                 bf16_weights=False, l2=None, step_outliers=0.0):
    """bf16_weights: round the seeded matrices to bf16-representable values first, so the oracle and the
    GPU's bf16 compute copy start from identical numbers and the comparison isolates the kernels.
    step_outliers: fraction of a gradient's elements that may pass the per-element step bound (by at most 4x); zero except
    for the 16-layer model, whose caller says why."""
    from eisen_amd import hip
    weights = gen.lm_weights(seed, std=0.02, perturb_norm=perturb_norm, **cfg)
    if bf16_weights:
        weights = [(n, hip.round_bf16(w) if w.ndim == 2 else w) for n, w in weights]
    gg, lm, og, olm = _build_pair(ctx, cfg, weights, precision)
    lm.set_fused(fused)
    opt, oopt = G.AdamW(gg, lm.params(), 1e-3), R.AdamW(og, olm.params(), 1e-3)
    opt.config(1e-3, 0.9, 0.95, 1e-8, 0.1, clip)
    oopt.config(1e-3, 0.9, 0.95, 1e-8, 0.1, clip)
    for step in range(steps):
        opt.zero_grad()
        oopt.zero_grad()
        for micro in range(accum):
            x, y = gen.lm_batch(1000 * seed + 10 * step + micro, mb, seq, cfg["vocab"], dist)
            lg, lo = lm.micro_step(x, y), olm.micro_step(x, y)
            assert abs(lg - lo) <= (1e-4 if precision == G.FP32 else 1e-2) * abs(lo), (lg, lo)
            assert gg.num_tensors() == len(weights) and gg.tape_len() == 0
        for pid, (name, _) in enumerate(weights):
            # the embedding gradient is row-sparse (untouched rows exactly zero, Zipf-hot rows large): per-row scale
            assert_close(gg.sync_grad_to_cpu(pid), og.grad(pid), rtol_grad, f"step {step} grad {name}", row_scale=(name == "embed"), l2=l2, step=(precision != G.FP32),
                         step_outliers=step_outliers)
        opt.step()
        oopt.step()
        for pid, (name, w) in enumerate(weights):
            got, exp = gg.sync_to_cpu(pid), og.data(pid)
            if precision == G.FP32:
                # a gradient element near zero turns its own rounding into an O(lr) change of the
                # normalised update: bound the worst element by 0.2*lr, the bulk tightly
                diff = np.abs(got - exp)
                assert diff.max() <= 0.2 * 1e-3 and diff.mean() <= 1e-6, name
            else:
                assert np.abs(got - exp).max() <= 2.1e-3, name            # every update is at most ~lr(1+wd|w|)
            og.load_tensor_data(pid, got)                                  # next step starts from identical weights
        for i in range(len(weights)):                                      # and identical moments
            m, v = opt.moments(i)
            om, ov = oopt.moments(i)
            assert_close(m, om, rtol_grad, f"m[{i}]", row_scale=(i == 0), l2=l2, step=(precision != G.FP32), step_outliers=step_outliers)
            np.ctypeslib.as_array(R.lib.ref_adamw_m(oopt.h, i), (m.size,))[:] = m
            np.ctypeslib.as_array(R.lib.ref_adamw_v(oopt.h, i), (v.size,))[:] = v
    return gg, lm, opt


def test_config1_f32_train_step_matches_oracle(ctx):
    """Config 1: vocab 256, d 64, 2 layers, 4 heads (head_dim 16, no GQA), ffn 256, B2 S32, untied, f32.
    Loss, every gradient and every updated weight vs the CPU oracle, rtol 1e-4; two optimiser steps."""
    cfg = dict(vocab=256, hidden=64, heads=4, kv_heads=4, ffn=256, layers=2, tie=False)
    _train_steps(ctx, cfg, G.FP32, 2, 32, steps=2, accum=1, rtol_grad=1e-4)


def test_config1_f32_unfused_chain_and_accumulation(ctx):
    """Same model through the reference's materialised attention chain (reshape/transpose/repeat_kv/
    bmm/mul/add/softmax/bmm), GQA 4:2, two accumulated micro-batches, gradient clipping on."""
    cfg = dict(vocab=256, hidden=64, heads=4, kv_heads=2, ffn=256, layers=2, tie=False)
    _train_steps(ctx, cfg, G.FP32, 2, 32, steps=1, accum=2, rtol_grad=1e-4, fused=False, clip=0.05)
    _train_steps(ctx, cfg, G.FP32, 2, 32, steps=1, accum=2, rtol_grad=1e-4, fused=True, clip=0.05)


def test_tied_embeddings_f32(ctx):
    cfg = dict(vocab=128, hidden=64, heads=4, kv_heads=2, ffn=128, layers=1, tie=True)
    _train_steps(ctx, cfg, G.FP32, 2, 24, steps=1, accum=2, rtol_grad=1e-4, dist="zipf")


def test_config4_architecture_bf16_mixed_step(ctx):
    """Config-4 architecture (vocab 8192, d 256, 6 layers, 8 q heads / 2 kv heads, head_dim 32, ffn 1024,
    tied, Zipf ids) at a micro-batch the oracle finishes in seconds (B2 S128); bf16 activations and
    matmuls, f32 master weights; gradients vs the f32 oracle at rtol 2e-2."""
    cfg = dict(vocab=8192, hidden=256, heads=8, kv_heads=2, ffn=1024, layers=6, tie=True)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 128, steps=1, accum=2, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)
    # weights as seeded (not bf16-representable): the rounding of the compute copy is part of the error
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 128, steps=1, accum=1, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, l2=2e-2)


def test_config5_block_shape_bf16_mixed_step(ctx):
    """One layer with config 5's head geometry (head_dim 64, 4:1 GQA) and an untied head at reduced width."""
    cfg = dict(vocab=1024, hidden=512, heads=8, kv_heads=2, ffn=1408, layers=1, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 128, steps=1, accum=1, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)


def test_equal_query_and_kv_heads_bf16_mixed_step(ctx):
    """No GQA (4 query heads, 4 K/V heads, head_dim 64): Q and K have one shape, so they leave one batched launch, both
    rotary-embedded by its epilogue, and V a plain one; and head_dim 32 with 512 tokens, where the three projections are
    whole 128 x 128 tiles."""
    cfg = dict(vocab=512, hidden=256, heads=4, kv_heads=4, ffn=512, layers=2, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 128, steps=1, accum=2, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)
    cfg = dict(vocab=512, hidden=256, heads=8, kv_heads=8, ffn=512, layers=1, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 256, steps=1, accum=1, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)


def test_wide_ffn_bf16_mixed_step(ctx):
    """2048 tokens through a 128 -> 4096 -> 128 feed-forward block: large enough for the kernel that forms gate, up and
    silu(gate) * up in one launch and for the wide-tile GEMMs behind it; head_dim 64, 2:1 GQA."""
    cfg = dict(vocab=256, hidden=128, heads=2, kv_heads=1, ffn=4096, layers=1, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 4, 512, steps=1, accum=1, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)


def test_deferred_weight_gradients_bf16_mixed_step(ctx):
    """Two layers whose gate and up projections are wide enough (256 -> 19200) for their weight gradients to wait for the
    Q/K/V group of the block and run with the Q, K, V and output projections' as one grouped launch; two accumulated
    micro-batches, so the launch also runs in its accumulating form."""
    cfg = dict(vocab=256, hidden=256, heads=4, kv_heads=2, ffn=19200, layers=2, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 128, steps=1, accum=2, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)


def test_biased_linear_and_parameter_operands_bf16_mixed(ctx):
    """Linear::forward with a bias (src/nn/linear.rs:88-93: matmul, then `g.add(out, bias)`), a product with a parameter
    vector and a sum with a parameter of the full shape, in mixed precision: the activations' gradients are bf16, the
    parameters' f32, and every parameter gradient is checked against the oracle."""
    from eisen_amd import hip
    M, K, N = 96, 64, 48
    vals = dict(x=hip.round_bf16(gen.normal(41, (M, K))), w=hip.round_bf16(gen.normal(42, (K, N), 0.2)), b=hip.round_bf16(gen.normal(43, (N,), 0.3)),
                gain=hip.round_bf16(1.0 + gen.normal(44, (N,), 0.2)), full=hip.round_bf16(gen.normal(45, (M, N), 0.3)))
    targets = gen.uniform_ids(46, (M,), N)
    grads = []
    for graph in (G.Graph(ctx, G.BF16_MIXED), R.Graph()):
        ids = {k: graph.alloc(v.shape, v) for k, v in vals.items()}
        graph.mark_params()
        for accum in range(2):  # the second pass adds into the f32 gradients
            h = graph.add(graph.matmul(ids["x"], ids["w"]), ids["b"])
            h = graph.mul(h, ids["gain"])
            h = graph.add(ids["full"], h)
            graph.backward(graph.cross_entropy(h, targets))
            graph.clear_activations()
        grads.append({k: (graph.sync_grad_to_cpu(i) if isinstance(graph, G.Graph) else graph.grad(i)) for k, i in ids.items()})
        if isinstance(graph, G.Graph):
            graph.close()
    for k in vals:
        assert_close(grads[0][k], grads[1][k], 2e-2, f"grad {k}", step=True)  # five bf16 ops composed


def test_head_dim_without_a_fused_kernel_bf16_mixed_step(ctx):
    """head_dim 96 in mixed precision: the bf16 attention kernels cover 32, 64 and 128, so the block takes the reference's
    materialised chain (rope, transposes, repeat_kv, bmm, scale, mask, softmax, bmm) while everything around it stays fused."""
    cfg = dict(vocab=128, hidden=192, heads=2, kv_heads=1, ffn=256, layers=1, tie=False)
    _train_steps(ctx, cfg, G.BF16_MIXED, 2, 64, steps=1, accum=2, rtol_grad=2e-2, dist="zipf", perturb_norm=0.0, bf16_weights=True)


def test_config5_layers_fused_path_matches_the_reference_chain(ctx):
    """Two layers at config 5's real width and micro-batch (d 2048, 32 q / 8 kv heads, ffn 5632, 4 x 1024 tokens): the fused
    path (grouped and deferred weight gradients, SwiGLU inside the GEMMs, side stream, rotary embedding inside attention)
    against the reference's op-by-op chain built from the individually oracle-checked kernels, same weights, two
    accumulated micro-batches.  The oracle itself would need minutes at this size."""
    from eisen_amd import hip
    cfg = dict(vocab=1024, hidden=2048, heads=32, kv_heads=8, ffn=5632, layers=2, tie=False)
    weights = [(n, hip.round_bf16(w) if w.ndim == 2 else w) for n, w in gen.lm_weights(3, std=0.02, perturb_norm=0.05, **cfg)]
    grads, losses = [], []
    for fused in (True, True, False):  # the fused path twice: the same bits both times (no atomics, ordered streams)
        gg = G.Graph(ctx, G.BF16_MIXED)
        lm = G.TransformerLM(gg, **cfg)
        for pid, (_, w) in enumerate(weights):
            gg.load_tensor_data(pid, w)
        gg.mark_params()
        lm.set_fused(fused)
        ls = []
        for micro in range(2):
            x, y = gen.lm_batch(3000 + micro, 4, 1024, cfg["vocab"], "zipf")
            ls.append(lm.micro_step(x, y))
        losses.append(ls)
        grads.append([gg.sync_grad_to_cpu(pid) for pid in range(len(weights))])
        gg.close()
    assert losses[0] == losses[1]
    for a, b in zip(losses[0], losses[2]):
        assert abs(a - b) <= 2e-3 * abs(b), losses
    for pid, (name, _) in enumerate(weights):
        assert np.array_equal(grads[0][pid], grads[1][pid]), f"grad {name} differs between two runs of the fused path"
        assert_close(grads[0][pid], grads[2][pid], 2e-2, f"grad {name}", row_scale=(name == "embed"), step=True)


def test_grad_accumulation_invariants_on_gpu(ctx):
    # tests/test_grad_accum.rs: additivity (:59-98), g_accum = N g_full (:108-166), clear_activations keeps
    # parameter gradients, zero_grad, tape emptied, tensor count back at the watermark
    cfg = dict(vocab=64, hidden=32, heads=4, kv_heads=2, ffn=64, layers=1, tie=False)
    gg = G.Graph(ctx, G.FP32)
    lm = G.TransformerLM(gg, **cfg)
    gg.mark_params()
    opt = G.AdamW(gg, lm.params(), 1e-2)
    x, y = gen.lm_batch(80, 2, 8, 64)
    opt.zero_grad()
    lm.micro_step(x, y)
    g1 = [gg.sync_grad_to_cpu(p) for p in lm.params()]
    assert gg.tape_len() == 0 and gg.num_tensors() == gg.num_params()
    lm.micro_step(x, y)
    for a, p in zip(g1, lm.params()):
        assert_close(gg.sync_grad_to_cpu(p), 2 * a, 1e-5, "additivity")
    opt.zero_grad()
    assert all(not gg.sync_grad_to_cpu(p).any() for p in lm.params())
    lm.micro_step(x, y)
    for a, p in zip(g1, lm.params()):
        assert np.array_equal(gg.sync_grad_to_cpu(p), a)          # deterministic kernels: identical bits
    norm, coef = opt.clip_grad_norm(1e-3)
    exact = np.sqrt(sum((a.astype(np.float64) ** 2).sum() for a in g1))
    assert abs(norm - exact) <= 1e-5 * exact and abs(coef - 1e-3 / (exact + 1e-6)) <= 1e-5 * coef
    norm2, coef2 = opt.clip_grad_norm(1.0)
    assert abs(norm2 - 1e-3) <= 1e-5 and coef2 == 1.0
    assert abs(gg.cosine_lr(1e-3, 1e-4, 10, 110, 60) - R.cosine_lr(1e-3, 1e-4, 10, 110, 60)) < 1e-9


def test_reference_initialisers(ctx):
    """Linear::new (seed-42 LCG + Box-Muller, std 0.02) and Embedding::new (seed-84 LCG, +-0.02): the
    integer streams are exact, so the values can be recomputed here."""
    gg = G.Graph(ctx, G.FP32)
    lm = G.TransformerLM(gg, 16, 8, 2, 1, 16, 1, False)
    emb = gg.sync_to_cpu(0).reshape(-1)
    seed, exp = 84, []
    for _ in range(emb.size):
        seed = (seed * 1664525 + 1013904223) % 2 ** 32
        exp.append((np.float32(seed) / np.float32(2 ** 32 - 1) * np.float32(2) - np.float32(1)) * np.float32(0.02))
    assert np.allclose(emb, np.array(exp, np.float32), rtol=1e-6, atol=1e-9)
    wq = gg.sync_to_cpu(2)
    assert wq.shape == (8, 8) and abs(wq.std() - 0.02) < 0.01 and np.array_equal(wq, gg.sync_to_cpu(5))   # same seed per layer
    assert lm.params() == [0, 1, 2, 3, 4, 5, 6, 8, 9, 7, 10, 11]


# ---- weights out: raw checkpoint and safetensors export ---------------------------------------

@pytest.mark.parametrize("precision,tie", [(G.FP32, False), (G.BF16_MIXED, True)])
def test_checkpoint_and_safetensors_export(ctx, tmp_path, precision, tie):
    from safetensors.numpy import load_file

    from eisen_amd import io as IO
    from oracle import io_ref as IR
    gr = G.Graph(ctx, precision)
    lm = G.TransformerLM(gr, vocab=48, hidden=32, heads=4, kv_heads=2, ffn=64, layers=2, tie=tie)
    gr.mark_params()  # everything allocated so far is a parameter (examples/train_llm.rs calls it after building the model)
    # tensor-id (construction) order, the order of the raw checkpoint; Module::params() lists the FFN weights
    # differently (src/nn/transformer.rs:57-66), which is why the reference's own save/load pair does not round-trip
    params = sorted(lm.params())
    arch = dict(vocab=48, hidden=32, heads=4, kv_heads=2, ffn=64, layers=2, tie=tie)
    weights = [w for _, w in gen.lm_weights(77, perturb_norm=0.1, **arch)]
    shapes = [s for _, s in gen.lm_param_shapes(**arch)]
    assert len(params) == len(weights)
    for pid, w in zip(params, weights):
        gr.load_tensor_data(pid, w)
    # raw checkpoint: every parameter in tensor-id order, f32 LE (examples/train_llm.rs:93-105)
    ck = tmp_path / "model.bin"
    IO.save_weights(gr, ck)
    assert ck.read_bytes() == IR.save_weights_bytes(weights)
    # and back (examples/chat_cli.rs:161-180) into a second model
    lm2 = G.TransformerLM(gr, vocab=48, hidden=32, heads=4, kv_heads=2, ffn=64, layers=2, tie=tie)
    assert IO.load_weights(gr, sorted(lm2.params()), ck) == sum(w.size for w in weights)
    for pid, w in zip(sorted(lm2.params()), weights):
        assert np.array_equal(gr.sync_to_cpu(pid).reshape(-1), w.reshape(-1))
    ck.write_bytes(ck.read_bytes()[:-8])
    with pytest.raises(EisenHipError, match="truncated"):
        IO.load_weights(gr, lm2.params(), ck)
    # safetensors: byte-identical to the restated writer, and readable by the safetensors library
    st = tmp_path / "model.safetensors"
    IO.write_safetensors(gr, lm, st)
    names = ["model.embed_tokens.weight"]
    for i in range(2):
        names += [f"model.layers.{i}.{n}.weight" for n in ("input_layernorm", "self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                                            "self_attn.o_proj", "post_attention_layernorm", "mlp.gate_proj", "mlp.up_proj",
                                                            "mlp.down_proj")]
    names += ["model.norm.weight"] + ([] if tie else ["lm_head.weight"])
    assert len(names) == len(weights)
    named = [(n, w.reshape(s)) for n, w, s in zip(names, weights, shapes)]
    assert st.read_bytes() == IR.safetensors_bytes(named)
    loaded = load_file(str(st))
    assert sorted(loaded) == sorted(names)
    for n, w in named:
        want = w if (w.ndim != 2 or n == "model.embed_tokens.weight") else w.T
        assert loaded[n].dtype == np.float32 and np.array_equal(loaded[n], want)
    lm.close(); lm2.close(); gr.close()
