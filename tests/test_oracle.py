"""Pins the CPU oracle (oracle/eisen_cpu_ref.c) without running the reference.

Each oracle function is checked against (1) the golden vectors the reference's own tests
hold (file:line cited per test), and (2) what the mathematics fixes: library routines it
must reduce to (torch in float64 with autograd), closed forms, and invariants -- chosen so
that a dropped term, a wrong sign/index or a transposed operand fails.
"""
import math

import numpy as np
import pytest
import torch

from oracle import cpu_ref as R
from tests import gen

torch.manual_seed(0)


def t64(a, grad=False):
    return torch.tensor(np.asarray(a), dtype=torch.float64, requires_grad=grad)


def close(a, b, rtol=1e-5, atol=1e-6):
    np.testing.assert_allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=rtol, atol=atol)


# ---------------------------------------------------------------------------
# golden vectors held by the reference's tests
# ---------------------------------------------------------------------------

def test_matmul_kat_reference():
    # tests/gpu_kernels.rs:79-103
    g = R.Graph()
    a = g.alloc((2, 3), [1, 2, 3, 4, 5, 6])
    b = g.alloc((3, 2), [7, 8, 9, 1, 2, 3])
    c = g.matmul(a, b)
    assert g.data(c).reshape(-1).tolist() == [31.0, 19.0, 85.0, 55.0]
    g.backward(c)
    assert g.grad(a).reshape(-1).tolist() == [15.0, 10.0, 5.0, 15.0, 10.0, 5.0]
    assert g.grad(b).reshape(-1).tolist() == [5.0, 5.0, 7.0, 7.0, 9.0, 9.0]


def test_add_mul_kat_reference():
    # tests/gpu_kernels.rs:27-41 and :52-67
    g = R.Graph()
    a = g.alloc((2, 2), [1, 2, 3, 4])
    b = g.alloc((2, 2), [0.5, 1.5, 2.5, 3.5])
    c = g.add(a, b)
    assert g.data(c).reshape(-1).tolist() == [1.5, 3.5, 5.5, 7.5]
    g.backward(c)
    assert g.grad(a).reshape(-1).tolist() == [1.0] * 4 and g.grad(b).reshape(-1).tolist() == [1.0] * 4
    g = R.Graph()
    a = g.alloc((3,), [2, -3, 4])
    b = g.alloc((3,), [5, 2, -1])
    c = g.mul(a, b)
    assert g.data(c).tolist() == [10.0, -6.0, -4.0]
    g.backward(c)
    assert g.grad(a).tolist() == [5.0, 2.0, -1.0] and g.grad(b).tolist() == [2.0, -3.0, 4.0]


def test_phase1_broadcast_transpose_max_sum():
    # tests/phase1.rs:4-45
    g = R.Graph()
    a = g.alloc((2, 3), [1, 2, 3, 4, 5, 6])
    b = g.alloc((1, 3), [10, 20, 30])
    c = g.add(a, b)
    d = g.transpose(c, 0, 1)
    e = g.max(d, 1)
    f = g.sum(e, 0)
    assert g.shape(f) == () and g.data(f).reshape(-1)[0] == 75.0
    g.backward(f)
    assert g.grad(a).reshape(-1).tolist() == [0, 0, 0, 1, 1, 1]
    assert g.grad(b).reshape(-1).tolist() == [1, 1, 1]


def test_sum_max_kat_reference():
    # tests/gpu_kernels.rs:301-331
    g = R.Graph()
    a = g.alloc((2, 3), [1, 2, 3, 4, 9, 6])
    s = g.sum(a, 1)
    assert g.data(s).tolist() == [6.0, 19.0]
    g.backward(s)
    assert g.grad(a).reshape(-1).tolist() == [1.0] * 6
    g = R.Graph()
    a = g.alloc((2, 3), [1, 2, 3, 4, 9, 6])
    m = g.max(a, 1)
    assert g.data(m).tolist() == [3.0, 9.0]
    g.backward(m)
    assert g.grad(a).reshape(-1).tolist() == [0, 0, 1, 0, 1, 0]


def test_silu_closed_form_reference():
    # tests/gpu_kernels.rs:114-152: silu(x) = x*sigmoid(x); d = sig*(1+x*(1-sig)), 1e-5
    x = np.array([-2.0, -1.0, 0.0, 1.0, 2.0, 5.5, -7.25], np.float32)
    sig = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    close(R.silu_fwd(x), x * sig, 1e-5, 1e-6)
    close(R.silu_bwd(x, np.ones_like(x)), sig * (1 + x * (1 - sig)), 1e-5, 1e-6)


def test_gather_kat_reference():
    # tests/gpu_kernels.rs:164-206 (collision on row 2) and tests/phase2_embedding.rs:37-43
    g = R.Graph()
    w = g.alloc((3, 2), [0.1, 0.2, 0.3, 0.4, 0.5, 0.6])
    idx = g.alloc((4,), [2, 0, 2, 1])
    c = g.gather(w, idx)
    close(g.data(c).reshape(-1), [0.5, 0.6, 0.1, 0.2, 0.5, 0.6, 0.3, 0.4], 0, 1e-7)
    g.backward(c)
    assert g.grad(w).reshape(-1).tolist() == [1, 1, 1, 1, 2, 2]
    g = R.Graph()
    w = g.alloc((4, 3), np.arange(12))
    idx = g.alloc((3,), [1, 1, 3])
    c = g.gather(w, idx)
    g.backward(c)
    assert g.grad(w).tolist() == [[0, 0, 0], [2, 2, 2], [0, 0, 0], [1, 1, 1]]


def test_cross_entropy_kat_reference():
    # tests/gpu_kernels.rs:262-289: loss ~0.27 (+-0.05), sign pattern of the gradient
    g = R.Graph()
    logits = g.alloc((2, 3), [2.0, 1.0, 0.1, 0.0, 3.0, 0.5])
    loss = g.cross_entropy(logits, [0, 1])
    lv = g.data(loss).reshape(-1)[0]
    assert abs(lv - 0.27) < 0.05
    g.backward(loss)
    gr = g.grad(logits).reshape(-1)
    assert gr[0] < 0 < gr[1] and gr[2] > 0 and gr[3] > 0 and gr[4] < 0 < gr[5]


def test_bmm_softmax_kat_reference():
    # tests/gpu_kernels.rs:344-376; rows sum to one: tests/cpu_attention_primitives.rs:14-19
    g = R.Graph()
    q = g.alloc((2, 2, 3), [1, 0, 1, 0, 1, 0, 1, 1, 1, 0, 0, 1])
    k = g.alloc((2, 2, 3), [1, 0, 1, 0, 1, 0, 1, 0, 0, 0, 0, 1])
    s = g.bmm(q, k, True)
    assert g.data(s).reshape(-1)[:4].tolist() == [2.0, 0.0, 0.0, 1.0]
    p = g.softmax(s)
    pv = g.data(p).reshape(-1)
    assert abs(pv[0] - 0.88079) < 1e-4 and abs(pv[1] - 0.11920) < 1e-4
    close(g.data(p).sum(-1), np.ones((2, 2)), 0, 1e-6)
    g.backward(p)
    assert np.any(g.grad(q) != 0) and np.any(g.grad(k) != 0)


def test_transpose_0213_grad_ones_reference():
    # tests/cpu_attention_primitives.rs:33-48
    g = R.Graph()
    t_in = g.alloc((1, 2, 2, 2), np.arange(1, 9))
    t = g.transpose_0213(t_in)
    assert g.shape(t) == (1, 2, 2, 2)
    s = g.sum(g.sum(g.sum(g.sum(t, 3), 2), 1), 0)
    g.backward(s)
    assert g.grad(t_in).reshape(-1).tolist() == [1.0] * 8


def test_flash_matches_unfused_reference():
    # tests/cpu_attention_primitives.rs:70-87 (1e-5) and tests/gpu_kernels.rs:403-429 (1e-4)
    for qd, kd, vd, shape in [
        ([1, 0, 0.5, 1], [1, 1, 0, 1], [0, 1, 2, 3], (1, 2, 2)),
        ([1, 0, 1, 0, 0, 1, 0, 1, 1, 1, 0, 0], [1, 0, 1, 0, 0, 1, 0, 1, 1, 1, 0, 0],
         [0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.1, 1.2], (1, 3, 4)),
    ]:
        g = R.Graph()
        g.set_no_grad(True)
        q, k, v = g.alloc(shape, qd), g.alloc(shape, kd), g.alloc(shape, vd)
        scale = np.float32(1.0) / np.sqrt(np.float32(shape[2]))
        s = g.bmm(q, k, True)
        sc = g.alloc((), [scale])
        p = g.softmax(g.mul(s, sc))
        ref = g.data(g.bmm(p, v, False))
        fl = g.data(g.flash_attention(q, k, v, scale, False))
        close(fl, ref, 0, 1e-5)


def test_rope_kat_reference():
    # tests/gpu_kernels.rs:485-513 and tests/cpu_attention_primitives.rs:56-60
    g = R.Graph()
    q = g.alloc((1, 2, 4), np.ones(8))
    r = g.rope(q, 4)
    rd = g.data(r).reshape(-1)
    assert rd[:4].tolist() == [1.0] * 4
    assert abs(rd[4] - (0.5403 - 0.8414)) < 1e-3 and abs(rd[5] - (0.5403 + 0.8414)) < 1e-3
    g.backward(r)
    qg = g.grad(q).reshape(-1)
    assert qg[:4].tolist() == [1.0] * 4
    assert abs(qg[4] - (0.5403 + 0.8414)) < 1e-3 and abs(qg[5] - (0.5403 - 0.8414)) < 1e-3


# ---------------------------------------------------------------------------
# what the mathematics fixes
# ---------------------------------------------------------------------------

def test_matmul_literal_vs_interchanged_bit_exact():
    a, b = gen.normal(1, (37, 129)), gen.normal(2, (129, 53))
    assert np.array_equal(R.matmul_fwd(a, b), R.matmul_fwd(a, b, literal=True))
    for threads in (1, 4):
        R.set_threads(threads)
        assert np.array_equal(R.matmul_fwd(a, b), R.matmul_fwd(a, b, literal=True))
    R.set_threads(8)


def test_matmul_family_vs_float64():
    a, b, go = gen.normal(3, (19, 40)), gen.normal(4, (40, 23)), gen.normal(5, (19, 23))
    close(R.matmul_fwd(a, b), a.astype(np.float64) @ b, 1e-5, 1e-5)
    ga, gb = R.matmul_bwd(a, b, go)
    close(ga, go.astype(np.float64) @ b.T, 1e-5, 1e-5)
    close(gb, a.T.astype(np.float64) @ go, 1e-5, 1e-5)
    # accumulation (+=) on a pre-filled grad
    ga2, gb2 = R.matmul_bwd(a, b, go, ga.copy(), gb.copy())
    close(ga2, 2 * ga, 1e-6, 1e-6)
    close(gb2, 2 * gb, 1e-6, 1e-6)
    bt = np.ascontiguousarray(b.T)
    close(R.matmul_trans_b_fwd(a, bt), a.astype(np.float64) @ b, 1e-5, 1e-5)
    ga, gbt = R.matmul_trans_b_bwd(a, bt, go)
    close(ga, go.astype(np.float64) @ b.T, 1e-5, 1e-5)
    close(gbt, (a.T.astype(np.float64) @ go).T, 1e-5, 1e-5)


@pytest.mark.parametrize("trans_b", [True, False])
def test_bmm_vs_float64(trans_b):
    a = gen.normal(6, (3, 5, 7))
    b = gen.normal(7, (3, 4, 7) if trans_b else (3, 7, 4))
    go = gen.normal(8, (3, 5, 4))
    bm = np.swapaxes(b, 1, 2) if trans_b else b
    close(R.bmm_fwd(a, b, trans_b), np.einsum("bmk,bkn->bmn", a.astype(np.float64), bm), 1e-5, 1e-5)
    ga, gb = R.bmm_bwd(a, b, go, trans_b)
    close(ga, np.einsum("bmn,bkn->bmk", go.astype(np.float64), bm), 1e-5, 1e-5)
    gbm = np.einsum("bmk,bmn->bkn", a.astype(np.float64), go)
    close(gb, np.swapaxes(gbm, 1, 2) if trans_b else gbm, 1e-5, 1e-5)


def test_softmax_vs_torch():
    x = gen.normal(9, (6, 33), 3.0)
    go = gen.normal(10, (6, 33))
    xt = t64(x, True)
    y = torch.softmax(xt, -1)
    y.backward(t64(go))
    out = R.softmax_fwd(x)
    close(out, y.detach(), 1e-5, 1e-7)
    close(R.softmax_bwd(out, go), xt.grad, 1e-4, 1e-6)


def test_cross_entropy_vs_torch_and_invariants():
    x = gen.normal(11, (9, 50), 2.0)
    t = gen.uniform_ids(12, (9,), 50)
    loss, gl, probs = R.cross_entropy(x, t)
    xt = t64(x, True)
    lt = torch.nn.functional.cross_entropy(xt, torch.tensor(t))
    lt.backward()
    close(loss, lt.item(), 1e-5, 1e-6)
    close(gl, xt.grad, 1e-4, 1e-7)
    close(gl.sum(-1), np.zeros(9), 0, 1e-6)                       # rows of dlogits sum to zero
    closed = np.mean(-np.log(probs[np.arange(9), t].astype(np.float64) + 1e-8))
    close(loss, closed, 1e-6, 0)                                  # -ln(p_t + 1e-8), mean over rows
    # the 1e-8 is visible when p_t is tiny: loss saturates at -ln(1e-8) instead of growing
    x2 = np.zeros((1, 4), np.float32)
    x2[0, 1] = 60.0
    loss2, _, _ = R.cross_entropy(x2, [0])
    assert abs(loss2 - (-math.log(1e-8))) < 1e-2
    # o_grad scales linearly
    _, gl3, _ = R.cross_entropy(x, t, 3.0)
    close(gl3, 3 * gl, 1e-6, 1e-9)


def test_cross_entropy_masked_vs_torch():
    x = gen.normal(13, (8, 20), 2.0)
    t = gen.uniform_ids(14, (8,), 20)
    t[[1, 5, 6]] = R.IGNORE_INDEX
    loss, gl = R.cross_entropy_masked(x, t)
    xt = t64(x, True)
    tt = torch.tensor(np.where(t < 0, -100, t))
    lt = torch.nn.functional.cross_entropy(xt, tt, ignore_index=-100)
    lt.backward()
    close(loss, lt.item(), 1e-5, 1e-6)
    close(gl, xt.grad, 1e-4, 1e-7)
    assert np.all(gl[[1, 5, 6]] == 0)
    # graph op: fallback and all-masked cases (src/graph/ops/reduction.rs:727-741)
    g = R.Graph()
    lid = g.alloc((8, 20), x)
    full = gen.uniform_ids(15, (8,), 20)
    a = g.data(g.cross_entropy_masked(lid, full)).reshape(-1)[0]
    b = g.data(g.cross_entropy(lid, full)).reshape(-1)[0]
    assert a == b
    n0 = g.tape_len()
    z = g.cross_entropy_masked(lid, np.full(8, R.IGNORE_INDEX))
    assert g.data(z).reshape(-1)[0] == 0.0 and g.tape_len() == n0


def test_transpose_0213_and_repeat_kv_vs_numpy():
    a = gen.normal(16, (2, 5, 3, 4))
    assert np.array_equal(R.transpose_0213_fwd(a), a.transpose(0, 2, 1, 3))
    go = gen.normal(17, (2, 3, 5, 4))
    assert np.array_equal(R.transpose_0213_bwd(go), go.transpose(0, 2, 1, 3))
    x = gen.normal(18, (2, 3, 5, 4))
    assert np.array_equal(R.repeat_kv_fwd(x, 4), np.repeat(x, 4, axis=1))       # repeat_interleave(dim=1)
    gq = gen.normal(19, (2, 12, 5, 4))
    close(R.repeat_kv_bwd(gq, 4), gq.reshape(2, 3, 4, 5, 4).astype(np.float64).sum(2), 1e-6, 1e-6)
    # summation order r ascending, bit-exact
    acc = np.zeros((2, 3, 5, 4), np.float32)
    for r in range(4):
        acc += gq.reshape(2, 3, 4, 5, 4)[:, :, r]
    assert np.array_equal(R.repeat_kv_bwd(gq, 4), acc)


def _rope_torch(x, head_dim):
    """Independent statement: interleaved pairs, theta = pos / 10000^(2p/hd)."""
    b, s, h = x.shape
    xr = x.reshape(b, s, h // head_dim, head_dim // 2, 2)
    p = torch.arange(head_dim // 2, dtype=torch.float64)
    pos = torch.arange(s, dtype=torch.float64)
    theta = pos[:, None] / (10000.0 ** (2 * p / head_dim))[None, :]
    c, sn = torch.cos(theta)[None, :, None, :], torch.sin(theta)[None, :, None, :]
    y0 = xr[..., 0] * c - xr[..., 1] * sn
    y1 = xr[..., 0] * sn + xr[..., 1] * c
    return torch.stack([y0, y1], -1).reshape(b, s, h)


def test_rope_vs_torch_and_invariants():
    x = gen.normal(20, (2, 9, 24))
    go = gen.normal(21, (2, 9, 24))
    xt = t64(x, True)
    y = _rope_torch(xt, 8)
    y.backward(t64(go))
    out = R.rope_fwd(x, 8)
    close(out, y.detach(), 1e-4, 1e-5)
    gx = R.rope_bwd(go, 8)
    close(gx, xt.grad, 1e-4, 1e-5)
    # rotation preserves each pair's norm; backward is the transpose (adjoint) of forward
    close((out.reshape(-1, 2) ** 2).sum(-1), (x.reshape(-1, 2) ** 2).sum(-1), 1e-5, 1e-6)
    close(np.vdot(out.astype(np.float64), go), np.vdot(x.astype(np.float64), gx), 1e-5, 1e-5)
    assert np.array_equal(out[:, 0], x[:, 0])                                   # position 0: identity


def test_rms_norm_vs_torch_and_invariants():
    x = gen.normal(22, (7, 48), 1.5)
    w = 1.0 + gen.normal(23, (48,), 0.2)
    go = gen.normal(24, (7, 48))
    eps = 1e-5
    xt, wt = t64(x, True), t64(w, True)
    y = torch.nn.functional.rms_norm(xt, (48,), wt, eps)
    y.backward(t64(go))
    out, rrms = R.rms_norm_fwd(x, w, eps)
    close(out, y.detach(), 1e-5, 1e-6)
    gx, gw = R.rms_norm_bwd(x, w, rrms, go)
    close(gx, xt.grad, 1e-4, 2e-6)
    close(gw, wt.grad, 1e-4, 2e-6)
    ss = (x.astype(np.float64) ** 2).sum(-1)
    close(((out / w) ** 2).mean(-1), ss / (ss + 48 * eps), 1e-5, 0)             # mean(y^2/w^2)


def test_attention_chain_vs_torch_autograd():
    """GQA attention core incl. reshape/transpose/repeat_kv/mask/scale vs torch float64 autograd."""
    B, S, H, KV, hd = 2, 7, 4, 2, 6
    d, kvd = H * hd, KV * hd
    x = gen.normal(30, (B, S, d), 0.7)
    ws = [gen.normal(31, (d, d), 0.2), gen.normal(32, (d, kvd), 0.2), gen.normal(33, (d, kvd), 0.2),
          gen.normal(34, (d, d), 0.2)]
    go = gen.normal(35, (B, S, d))
    g = R.Graph()
    xid = g.alloc(x.shape, x)
    wid = [g.alloc(w.shape, w) for w in ws]
    out = g.gqa_forward(H, KV, hd, *wid, xid, True)
    assert g.shape(out) == (B, S, d)
    # seed the output grad with `go` through a mul+sum reduction: loss = sum(out*go)
    gid = g.alloc(go.shape, go)
    prod = g.mul(out, gid)
    loss = g.sum(g.sum(g.sum(prod, 2), 1), 0)
    g.backward(loss)

    xt = t64(x, True)
    wt = [t64(w, True) for w in ws]
    q = _rope_torch(xt @ wt[0], hd).reshape(B, S, H, hd).transpose(1, 2)
    k = _rope_torch(xt @ wt[1], hd).reshape(B, S, KV, hd).transpose(1, 2).repeat_interleave(H // KV, 1)
    v = (xt @ wt[2]).reshape(B, S, KV, hd).transpose(1, 2).repeat_interleave(H // KV, 1)
    sc = (q @ k.transpose(-1, -2)) / math.sqrt(hd)
    sc = sc.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    ctx = (torch.softmax(sc, -1) @ v).transpose(1, 2).reshape(B, S, d)
    ot = ctx @ wt[3]
    (ot * t64(go)).sum().backward()
    close(g.data(out), ot.detach(), 1e-4, 1e-6)
    close(g.grad(xid), xt.grad, 2e-4, 2e-6)
    for i in range(4):
        close(g.grad(wid[i]), wt[i].grad, 2e-4, 2e-6)
    # no_grad path takes the flash forward (src/nn/attention.rs:335-336) and must agree
    g2 = R.Graph()
    g2.set_no_grad(True)
    xid2 = g2.alloc(x.shape, x)
    wid2 = [g2.alloc(w.shape, w) for w in ws]
    out2 = g2.gqa_forward(H, KV, hd, *wid2, xid2, True)
    close(g2.data(out2), g.data(out), 1e-5, 1e-6)
    assert g2.tape_len() == 0


def test_adamw_closed_form_and_torch():
    # first step from zero moments: bias corrections cancel -> w1 = w0(1-lr*wd) - lr*g/(|g|+eps)
    w0 = gen.normal(40, (64,))
    gr = gen.normal(41, (64,))
    w, m, v = w0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.95, 1e-8, 0.1
    R.adamw_update(w, gr, m, v, lr, b1, b2, eps, wd, 1)
    close(w, w0.astype(np.float64) * (1 - lr * wd) - lr * gr / (np.abs(gr.astype(np.float64)) + eps), 1e-5, 1e-7)
    # five steps vs torch.optim.AdamW (same algebra: decoupled decay, eps outside the corrected sqrt)
    wt = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.AdamW([wt], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    w, m, v = w0.copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    for t in range(1, 6):
        gt = gen.normal(100 + t, (64,))
        wt.grad = t64(gt)
        opt.step()
        R.adamw_update(w, gt, m, v, lr, b1, b2, eps, wd, t)
    close(w, wt.detach(), 2e-5, 1e-6)
    bc1, bc2 = R.adamw_bias_corrections(0.9, 0.95, 3)
    close([bc1, bc2], [1 / (1 - 0.9 ** 3), 1 / (1 - 0.95 ** 3)], 1e-6, 0)
    assert R.lib.ref_powi(2.0, 10) == 1024.0 and R.lib.ref_powi(3.0, 0) == 1.0


def test_clip_and_scheduler():
    g1, g2 = gen.normal(42, (100,)), gen.normal(43, (7, 9))
    norm, coef = R.grad_norm_clip_coef([g1, g2], 1.0)
    exact = math.sqrt((g1.astype(np.float64) ** 2).sum() + (g2.astype(np.float64) ** 2).sum())
    close(norm, exact, 1e-6, 0)
    close(coef, min(1.0, 1.0 / (exact + 1e-6)), 1e-6, 0)
    assert R.grad_norm_clip_coef([g1 * 1e-3], 1.0)[1] == 1.0
    # src/nn/scheduler.rs:45-55
    close(R.cosine_lr(1e-3, 1e-4, 10, 110, 0), 1e-4, 1e-6, 0)
    close(R.cosine_lr(1e-3, 1e-4, 10, 110, 9), 1e-3, 1e-6, 0)
    close(R.cosine_lr(1e-3, 1e-4, 10, 110, 60), 1e-4 + 0.5 * 9e-4, 1e-5, 0)
    close(R.cosine_lr(1e-3, 1e-4, 10, 110, 500), 1e-4, 1e-5, 0)


# ---------------------------------------------------------------------------
# the composed training step
# ---------------------------------------------------------------------------

class TorchLM(torch.nn.Module):
    """Independent float64 statement of the model in src/nn/transformer.rs (weights [in,out])."""

    def __init__(self, cfg, weights):
        super().__init__()
        self.cfg = cfg
        self.p = torch.nn.ParameterList([torch.nn.Parameter(t64(w)) for _, w in weights])

    def forward(self, ids):
        c = self.cfg
        H, KV, d = c["heads"], c["kv_heads"], c["hidden"]
        hd = d // H
        B, S = ids.shape
        it = iter(self.p)
        emb = next(it)
        h = emb[ids]
        mask = torch.triu(torch.ones(S, S, dtype=torch.bool), 1)
        for _ in range(c["layers"]):
            n1, wq, wk, wv, wo, n2, wg, wu, wd = (next(it) for _ in range(9))
            x = torch.nn.functional.rms_norm(h, (d,), n1, 1e-5)
            q = _rope_torch(x @ wq, hd).reshape(B, S, H, hd).transpose(1, 2)
            k = _rope_torch(x @ wk, hd).reshape(B, S, KV, hd).transpose(1, 2).repeat_interleave(H // KV, 1)
            v = (x @ wv).reshape(B, S, KV, hd).transpose(1, 2).repeat_interleave(H // KV, 1)
            sc = (q @ k.transpose(-1, -2)) / math.sqrt(hd)
            a = torch.softmax(sc.masked_fill(mask, float("-inf")), -1) @ v
            h = h + a.transpose(1, 2).reshape(B, S, d) @ wo
            x = torch.nn.functional.rms_norm(h, (d,), n2, 1e-5)
            h = h + (torch.nn.functional.silu(x @ wg) * (x @ wu)) @ wd
        h = torch.nn.functional.rms_norm(h, (d,), next(it), 1e-5)
        return h @ (emb.T if c["tie"] else next(it))


def _build(cfg, weights):
    g = R.Graph()
    lm = R.TransformerLM(g, **cfg)
    for (name, w), pid in zip(weights, range(g.num_tensors())):
        assert g.shape(pid) == w.shape, name
        g.load_tensor_data(pid, w)
    g.mark_params()
    return g, lm


@pytest.mark.parametrize("tie,kv", [(False, 4), (True, 2)])
def test_lm_train_step_vs_torch(tie, kv):
    """Config-1 architecture (vocab 256, d 64, 2 layers, 4 heads, ffn 256, B2 S32): loss, every
    gradient and every updated weight against torch float64 autograd + torch.optim.AdamW."""
    cfg = dict(vocab=256, hidden=64, heads=4, kv_heads=kv, ffn=256, layers=2, tie=tie)
    weights = gen.lm_weights(1, std=0.02, perturb_norm=0.05, **cfg)
    g, lm = _build(cfg, weights)
    opt = R.AdamW(g, lm.params(), 1e-3)
    opt.config(1e-3, 0.9, 0.95, 1e-8, 0.1)
    tm = TorchLM(cfg, weights)
    topt = torch.optim.AdamW(tm.parameters(), lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for step in range(2):
        opt.zero_grad()
        topt.zero_grad()
        losses = []
        for micro in range(2):                       # accumulation: grads sum, no 1/N (train_llm.rs:399-458)
            x, y = gen.lm_batch(50 + 10 * step + micro, 2, 32, 256)
            losses.append(lm.micro_step(x, y))
            tl = torch.nn.functional.cross_entropy(tm(torch.tensor(x)).reshape(-1, 256), torch.tensor(y))
            tl.backward()
            close(losses[-1], tl.item(), 1e-5, 0)
            assert g.num_tensors() == len(weights) and g.tape_len() == 0
        for pid, tp in zip(range(len(weights)), tm.parameters()):
            gr = g.grad(pid)
            scale = float(tp.grad.abs().max()) + 1e-12
            assert np.abs(gr - tp.grad.numpy()).max() <= 2e-4 * scale, weights[pid][0]
        opt.step()
        topt.step()
        # AdamW divides by sqrt(v): an element whose gradient is ~0 turns f32 rounding of the
        # gradient into an O(lr) difference, so bound the worst element by 0.2*lr and the mean tightly
        # (the update rule itself is pinned with identical gradients in test_adamw_closed_form_and_torch).
        for pid, tp in zip(range(len(weights)), tm.parameters()):
            diff = np.abs(g.data(pid) - tp.detach().numpy())
            assert diff.max() <= 0.2 * 1e-3 and diff.mean() <= 2e-7, weights[pid][0]
            with torch.no_grad():                     # next step starts from identical weights
                tp.copy_(t64(g.data(pid)))


def test_grad_accumulation_invariants():
    # tests/test_grad_accum.rs: additivity (:59-98), clear_activations keeps param grads,
    # tape emptied, tensor count back to the watermark, zero_grad, AdamW equal under accumulation (:484-538)
    cfg = dict(vocab=64, hidden=32, heads=4, kv_heads=2, ffn=64, layers=1, tie=False)
    weights = gen.lm_weights(2, **cfg)
    x, y = gen.lm_batch(60, 2, 8, 64)
    g, lm = _build(cfg, weights)
    lm.micro_step(x, y)
    g1 = [g.grad(p) for p in lm.params()]
    assert g.tape_len() == 0 and g.num_tensors() == len(weights)
    lm.micro_step(x, y)
    for a, p in zip(g1, lm.params()):
        close(g.grad(p), 2 * a, 1e-6, 1e-9)
    opt = R.AdamW(g, lm.params(), 1e-2)
    opt.zero_grad()
    assert all(not g.grad(p).any() for p in lm.params())
    # params order: emb, (norm1,q,k,v,o,norm2,up,down,gate), norm_f, lm_head (src/nn/transformer.rs:57-66,198-210)
    assert lm.params() == [0, 1, 2, 3, 4, 5, 6, 8, 9, 7, 10, 11]
    # clipping: scale applied once norm > max
    lm.micro_step(x, y)
    norm, coef = opt.clip_grad_norm(1e-3)
    exact = math.sqrt(sum((a.astype(np.float64) ** 2).sum() for a in g1))
    close(norm, exact, 1e-5, 0)
    close(coef, 1e-3 / (exact + 1e-6), 1e-5, 0)
    norm2, _ = opt.clip_grad_norm(1.0)
    close(norm2, 1e-3, 1e-3, 0)
