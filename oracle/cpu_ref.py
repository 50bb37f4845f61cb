"""ctypes binding of the CPU oracle (oracle/eisen_cpu_ref.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker / the timed CPU baseline.  The shipped
package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libeisen_cpu_ref.so")

IGNORE_INDEX = -1  # usize::MAX reinterpreted as int64

f32p = C.POINTER(C.c_float)
i64p = C.POINTER(C.c_int64)
szp = C.POINTER(C.c_size_t)
intp = C.POINTER(C.c_int)


def build(force=False):
    """Compile the oracle with its Makefile (gcc)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_sz, _f, _i, _vp = C.c_size_t, C.c_float, C.c_int, C.c_void_p

_sig("ref_set_threads", None, _i)
_sig("ref_get_threads", _i)
_sig("ref_powi", _f, _f, _i)
for _n in ("ref_matmul_fwd", "ref_matmul_fwd_literal", "ref_matmul_trans_b_fwd"):
    _sig(_n, None, f32p, f32p, f32p, _sz, _sz, _sz)
for _n in ("ref_matmul_bwd", "ref_matmul_trans_b_bwd"):
    _sig(_n, None, f32p, f32p, f32p, f32p, f32p, _sz, _sz, _sz)
_sig("ref_bmm_fwd", None, f32p, f32p, f32p, _sz, _sz, _sz, _sz, _i)
_sig("ref_bmm_bwd", None, f32p, f32p, f32p, f32p, f32p, _sz, _sz, _sz, _sz, _i)
_sig("ref_silu_fwd", None, f32p, f32p, _sz)
_sig("ref_silu_bwd", None, f32p, f32p, f32p, _sz)
_sig("ref_softmax_fwd", None, f32p, f32p, _sz, _sz)
_sig("ref_softmax_bwd", None, f32p, f32p, f32p, _sz, _sz)
_sig("ref_cross_entropy_fwd", _f, f32p, i64p, f32p, _sz, _sz)
_sig("ref_cross_entropy_bwd", None, f32p, i64p, _f, f32p, _sz, _sz)
_sig("ref_cross_entropy_masked_fwd", _f, f32p, i64p, f32p, _sz, _sz, _f)
_sig("ref_cross_entropy_masked_bwd", None, f32p, i64p, _f, f32p, _sz, _sz, _f)
_sig("ref_transpose_0213_fwd", None, f32p, f32p, _sz, _sz, _sz, _sz)
_sig("ref_transpose_0213_bwd", None, f32p, f32p, _sz, _sz, _sz, _sz)
_sig("ref_gather_fwd", None, f32p, f32p, f32p, _sz, _sz)
_sig("ref_gather_bwd", None, f32p, f32p, f32p, _sz, _sz)
_sig("ref_rope_fwd", None, f32p, f32p, _sz, _sz, _sz, _sz)
_sig("ref_rope_bwd", None, f32p, f32p, _sz, _sz, _sz, _sz)
_sig("ref_rms_norm_fwd", None, f32p, f32p, f32p, f32p, _sz, _sz, _f)
_sig("ref_rms_norm_bwd", None, f32p, f32p, f32p, f32p, f32p, f32p, _sz, _sz)
_sig("ref_repeat_kv_fwd", None, f32p, f32p, _sz, _sz, _sz, _sz, _sz)
_sig("ref_repeat_kv_bwd", None, f32p, f32p, _sz, _sz, _sz, _sz, _sz)
_sig("ref_flash_attention_fwd", None, f32p, f32p, f32p, f32p, _sz, _sz, _sz, _sz, _f, _i)
_sig("ref_adamw_bias_corrections", None, _f, _f, _i, f32p, f32p)
_sig("ref_adamw_update", None, f32p, f32p, f32p, f32p, _sz, _f, _f, _f, _f, _f, _f, _f)
_sig("ref_sum_squares_f64", C.c_double, f32p, _sz, C.c_double)
_sig("ref_clip_coef", _f, C.c_double, _f, f32p)
_sig("ref_cosine_lr", _f, _f, _f, _sz, _sz, _sz)

_sig("ref_graph_new", _vp)
_sig("ref_graph_free", None, _vp)
_sig("ref_alloc", _i, _vp, szp, _i, f32p)
_sig("ref_data", f32p, _vp, _i)
_sig("ref_grad", f32p, _vp, _i)
_sig("ref_numel", _sz, _vp, _i)
_sig("ref_rank", _i, _vp, _i)
_sig("ref_dim", _sz, _vp, _i, _i)
_sig("ref_num_tensors", _i, _vp)
_sig("ref_tape_len", _i, _vp)
_sig("ref_set_no_grad", None, _vp, _i)
_sig("ref_mark_params", None, _vp)
_sig("ref_load_tensor_data", None, _vp, _i, f32p, _sz)
_sig("ref_reinterpret_shape", None, _vp, _i, szp, _i)
_sig("ref_restore_save_point", None, _vp, _i)
_sig("ref_clear_activations", None, _vp)
_sig("ref_zero_grad", None, _vp, _i)
for _n in ("ref_add", "ref_mul", "ref_matmul", "ref_matmul_trans_b", "ref_gather"):
    _sig(_n, _i, _vp, _i, _i)
_sig("ref_mul_ex", _i, _vp, _i, _i, _i)
for _n in ("ref_silu", "ref_softmax", "ref_transpose_0213"):
    _sig(_n, _i, _vp, _i)
_sig("ref_bmm", _i, _vp, _i, _i, _i)
_sig("ref_cross_entropy", _i, _vp, _i, i64p)
_sig("ref_cross_entropy_masked", _i, _vp, _i, i64p)
_sig("ref_reshape", _i, _vp, _i, szp, _i)
_sig("ref_rope", _i, _vp, _i, _sz)
_sig("ref_rms_norm", _i, _vp, _i, _i, _f)
_sig("ref_repeat_kv", _i, _vp, _i, _sz)
_sig("ref_flash_attention", _i, _vp, _i, _i, _i, _f, _i)
_sig("ref_sum", _i, _vp, _i, _i)
_sig("ref_max", _i, _vp, _i, _i)
_sig("ref_transpose", _i, _vp, _i, _i, _i)
_sig("ref_backward", None, _vp, _i)
_sig("ref_lm_new", _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _i)
_sig("ref_lm_free", None, _vp)
_sig("ref_lm_params", _i, _vp, intp)
_sig("ref_gqa_forward", _i, _vp, _sz, _sz, _sz, _i, _i, _i, _i, _i, _i)
_sig("ref_lm_forward", _i, _vp, _vp, _i)
_sig("ref_lm_micro_step", _f, _vp, _vp, f32p, i64p, _sz, _sz)
_sig("ref_adamw_new", _vp, _vp, intp, _i, _f)
_sig("ref_adamw_free", None, _vp)
_sig("ref_adamw_config", None, _vp, _f, _f, _f, _f, _f, _f)
_sig("ref_adamw_m", f32p, _vp, _i)
_sig("ref_adamw_v", f32p, _vp, _i)
_sig("ref_adamw_t", _i, _vp)
_sig("ref_adamw_last_grad_norm", _f, _vp)
_sig("ref_adamw_zero_grad", None, _vp, _vp)
_sig("ref_adamw_clip_grad_norm", _f, _vp, _vp, _f, f32p)
_sig("ref_adamw_step", None, _vp, _vp)

lib = _lib


def set_threads(n):
    _lib.ref_set_threads(int(n))


def get_threads():
    return int(_lib.ref_get_threads())


def fp(a):
    """float32 C-contiguous numpy array -> float*."""
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(f32p)


def ip(a):
    assert a.dtype == np.int64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(i64p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _shape(shape):
    arr = (C.c_size_t * max(len(shape), 1))(*shape)
    return arr, len(shape)


# ---------------------------------------------------------------------------
# stateless wrappers: numpy in, numpy out
# ---------------------------------------------------------------------------

def matmul_fwd(a, b, literal=False):
    a, b = _f32(a), _f32(b)
    m, k = a.shape
    n = b.shape[1]
    out = np.empty((m, n), np.float32)
    (_lib.ref_matmul_fwd_literal if literal else _lib.ref_matmul_fwd)(fp(a), fp(b), fp(out), m, k, n)
    return out


def matmul_bwd(a, b, go, ga=None, gb=None):
    a, b, go = _f32(a), _f32(b), _f32(go)
    m, k = a.shape
    n = b.shape[1]
    ga = np.zeros_like(a) if ga is None else ga
    gb = np.zeros_like(b) if gb is None else gb
    _lib.ref_matmul_bwd(fp(a), fp(b), fp(go), fp(ga), fp(gb), m, k, n)
    return ga, gb


def matmul_trans_b_fwd(a, b):
    a, b = _f32(a), _f32(b)
    m, k = a.shape
    n = b.shape[0]
    out = np.empty((m, n), np.float32)
    _lib.ref_matmul_trans_b_fwd(fp(a), fp(b), fp(out), m, k, n)
    return out


def matmul_trans_b_bwd(a, b, go):
    a, b, go = _f32(a), _f32(b), _f32(go)
    m, k = a.shape
    n = b.shape[0]
    ga, gb = np.zeros_like(a), np.zeros_like(b)
    _lib.ref_matmul_trans_b_bwd(fp(a), fp(b), fp(go), fp(ga), fp(gb), m, k, n)
    return ga, gb


def bmm_fwd(a, b, trans_b):
    a, b = _f32(a), _f32(b)
    batch, m, k = a.shape
    n = b.shape[1] if trans_b else b.shape[2]
    out = np.empty((batch, m, n), np.float32)
    _lib.ref_bmm_fwd(fp(a), fp(b), fp(out), batch, m, k, n, int(trans_b))
    return out


def bmm_bwd(a, b, go, trans_b):
    a, b, go = _f32(a), _f32(b), _f32(go)
    batch, m, k = a.shape
    n = b.shape[1] if trans_b else b.shape[2]
    ga, gb = np.zeros_like(a), np.zeros_like(b)
    _lib.ref_bmm_bwd(fp(a), fp(b), fp(go), fp(ga), fp(gb), batch, m, k, n, int(trans_b))
    return ga, gb


def silu_fwd(x):
    x = _f32(x)
    out = np.empty_like(x)
    _lib.ref_silu_fwd(fp(x), fp(out), x.size)
    return out


def silu_bwd(x, go):
    x, go = _f32(x), _f32(go)
    gx = np.zeros_like(x)
    _lib.ref_silu_bwd(fp(x), fp(go), fp(gx), x.size)
    return gx


def softmax_fwd(x):
    x = _f32(x)
    n = x.shape[-1]
    out = np.empty_like(x)
    _lib.ref_softmax_fwd(fp(x), fp(out), x.size // n, n)
    return out


def softmax_bwd(out, go):
    out, go = _f32(out), _f32(go)
    n = out.shape[-1]
    gx = np.zeros_like(out)
    _lib.ref_softmax_bwd(fp(out), fp(go), fp(gx), out.size // n, n)
    return gx


def cross_entropy(logits, targets, o_grad=1.0):
    """Returns (mean loss, dlogits, probs)."""
    logits = _f32(logits)
    targets = np.ascontiguousarray(targets, dtype=np.int64)
    rows, classes = logits.shape
    probs = np.empty_like(logits)
    loss = _lib.ref_cross_entropy_fwd(fp(logits), ip(targets), fp(probs), rows, classes)
    gl = np.zeros_like(logits)
    _lib.ref_cross_entropy_bwd(fp(probs), ip(targets), float(o_grad), fp(gl), rows, classes)
    return float(loss), gl, probs


def cross_entropy_masked(logits, targets, o_grad=1.0):
    logits = _f32(logits)
    targets = np.ascontiguousarray(targets, dtype=np.int64)
    rows, classes = logits.shape
    valid = int((targets != IGNORE_INDEX).sum())
    if valid == rows:
        loss, gl, _ = cross_entropy(logits, targets, o_grad)
        return loss, gl
    if valid == 0:
        return 0.0, np.zeros_like(logits)
    normalizer = np.float32(1.0) / np.float32(valid)
    probs = np.empty_like(logits)
    loss = _lib.ref_cross_entropy_masked_fwd(fp(logits), ip(targets), fp(probs), rows, classes, float(normalizer))
    gl = np.zeros_like(logits)
    _lib.ref_cross_entropy_masked_bwd(fp(probs), ip(targets), float(o_grad), fp(gl), rows, classes, float(normalizer))
    return float(loss), gl


def transpose_0213_fwd(a):
    a = _f32(a)
    b, s, h, d = a.shape
    out = np.empty((b, h, s, d), np.float32)
    _lib.ref_transpose_0213_fwd(fp(a), fp(out), b, s, h, d)
    return out


def transpose_0213_bwd(go, ga=None):
    go = _f32(go)
    b, h, s, d = go.shape
    ga = np.zeros((b, s, h, d), np.float32) if ga is None else ga
    _lib.ref_transpose_0213_bwd(fp(go), fp(ga), b, s, h, d)
    return ga


def gather_fwd(w, idx):
    w, idx = _f32(w), _f32(idx)
    out = np.empty(idx.shape + (w.shape[1],), np.float32)
    _lib.ref_gather_fwd(fp(w), fp(idx), fp(out), idx.size, w.shape[1])
    return out


def gather_bwd(idx, go, vocab, gw=None):
    idx, go = _f32(idx), _f32(go)
    hidden = go.shape[-1]
    gw = np.zeros((vocab, hidden), np.float32) if gw is None else gw
    _lib.ref_gather_bwd(fp(idx), fp(go), fp(gw), idx.size, hidden)
    return gw


def rope_fwd(x, head_dim):
    x = _f32(x)
    b, s, h = x.shape
    out = np.empty_like(x)
    _lib.ref_rope_fwd(fp(x), fp(out), b, s, h, head_dim)
    return out


def rope_bwd(go, head_dim, ga=None):
    go = _f32(go)
    b, s, h = go.shape
    ga = np.zeros_like(go) if ga is None else ga
    _lib.ref_rope_bwd(fp(go), fp(ga), b, s, h, head_dim)
    return ga


def rms_norm_fwd(x, w, eps):
    x, w = _f32(x), _f32(w)
    dim = x.shape[-1]
    nv = x.size // dim
    out = np.empty_like(x)
    rrms = np.empty(nv, np.float32)
    _lib.ref_rms_norm_fwd(fp(x), fp(w), fp(out), fp(rrms), nv, dim, float(eps))
    return out, rrms


def rms_norm_bwd(x, w, rrms, go, gx=None, gw=None):
    x, w, rrms, go = _f32(x), _f32(w), _f32(rrms), _f32(go)
    dim = x.shape[-1]
    nv = x.size // dim
    gx = np.zeros_like(x) if gx is None else gx
    gw = np.zeros_like(w) if gw is None else gw
    _lib.ref_rms_norm_bwd(fp(x), fp(w), fp(rrms), fp(go), fp(gx), fp(gw), nv, dim)
    return gx, gw


def repeat_kv_fwd(x, repeats):
    x = _f32(x)
    b, kv, s, d = x.shape
    out = np.empty((b, kv * repeats, s, d), np.float32)
    _lib.ref_repeat_kv_fwd(fp(x), fp(out), b, kv, s, d, repeats)
    return out


def repeat_kv_bwd(go, repeats):
    go = _f32(go)
    b, qh, s, d = go.shape
    gin = np.zeros((b, qh // repeats, s, d), np.float32)
    _lib.ref_repeat_kv_bwd(fp(go), fp(gin), b, qh // repeats, s, d, repeats)
    return gin


def flash_attention_fwd(q, k, v, scale, causal):
    q, k, v = _f32(q), _f32(k), _f32(v)
    batch, m, d = q.shape
    n = k.shape[1]
    out = np.empty_like(q)
    _lib.ref_flash_attention_fwd(fp(q), fp(k), fp(v), fp(out), batch, m, n, d, float(scale), int(causal))
    return out


def adamw_bias_corrections(beta1, beta2, t):
    b1, b2 = C.c_float(), C.c_float()
    _lib.ref_adamw_bias_corrections(float(beta1), float(beta2), int(t), C.byref(b1), C.byref(b2))
    return b1.value, b2.value


def adamw_update(w, g, m, v, lr, beta1, beta2, eps, wd, t):
    """In-place on w, m, v (float32 arrays)."""
    bc1, bc2 = adamw_bias_corrections(beta1, beta2, t)
    _lib.ref_adamw_update(fp(w), fp(_f32(g)), fp(m), fp(v), w.size, lr, beta1, beta2, eps, wd, bc1, bc2)


def grad_norm_clip_coef(grads, max_norm):
    ss = 0.0
    for g in grads:
        g = _f32(g)
        ss = _lib.ref_sum_squares_f64(fp(g), g.size, ss)
    norm = C.c_float()
    coef = _lib.ref_clip_coef(ss, float(max_norm), C.byref(norm))
    return norm.value, coef


def cosine_lr(lr_max, lr_min, warmup, total, step):
    return _lib.ref_cosine_lr(lr_max, lr_min, warmup, total, step)


# ---------------------------------------------------------------------------
# Graph / tape mirror
# ---------------------------------------------------------------------------

class Graph:
    """Mirror of the reference's CPU `Graph` (src/graph/mod.rs) over the C oracle."""

    def __init__(self):
        self.h = _lib.ref_graph_new()

    def __del__(self):
        if getattr(self, "h", None):
            _lib.ref_graph_free(self.h)
            self.h = None

    def alloc(self, shape, data=None):
        sh, rank = _shape(tuple(shape))
        if data is None:
            return _lib.ref_alloc(self.h, sh, rank, None)
        d = _f32(data).reshape(-1)
        return _lib.ref_alloc(self.h, sh, rank, fp(d))

    def shape(self, i):
        return tuple(_lib.ref_dim(self.h, i, k) for k in range(_lib.ref_rank(self.h, i)))

    def data(self, i):
        n = _lib.ref_numel(self.h, i)
        return np.ctypeslib.as_array(_lib.ref_data(self.h, i), (n,)).reshape(self.shape(i)).copy()

    def grad(self, i):
        n = _lib.ref_numel(self.h, i)
        return np.ctypeslib.as_array(_lib.ref_grad(self.h, i), (n,)).reshape(self.shape(i)).copy()

    def load_tensor_data(self, i, data):
        d = _f32(data).reshape(-1)
        _lib.ref_load_tensor_data(self.h, i, fp(d), d.size)

    def num_tensors(self):
        return _lib.ref_num_tensors(self.h)

    def tape_len(self):
        return _lib.ref_tape_len(self.h)

    def set_no_grad(self, v):
        _lib.ref_set_no_grad(self.h, int(v))

    def mark_params(self):
        _lib.ref_mark_params(self.h)

    def clear_activations(self):
        _lib.ref_clear_activations(self.h)

    def zero_grad(self, i):
        _lib.ref_zero_grad(self.h, i)

    def reinterpret_shape(self, i, shape):
        sh, rank = _shape(tuple(shape))
        _lib.ref_reinterpret_shape(self.h, i, sh, rank)

    def add(self, a, b): return _lib.ref_add(self.h, a, b)
    def mul(self, a, b): return _lib.ref_mul(self.h, a, b)
    def mul_const(self, a, b): return _lib.ref_mul_ex(self.h, a, b, 1)
    def silu(self, a): return _lib.ref_silu(self.h, a)
    def matmul(self, a, b): return _lib.ref_matmul(self.h, a, b)
    def matmul_trans_b(self, a, b): return _lib.ref_matmul_trans_b(self.h, a, b)
    def bmm(self, a, b, trans_b): return _lib.ref_bmm(self.h, a, b, int(trans_b))
    def softmax(self, a): return _lib.ref_softmax(self.h, a)
    def transpose_0213(self, a): return _lib.ref_transpose_0213(self.h, a)
    def gather(self, w, idx): return _lib.ref_gather(self.h, w, idx)
    def rope(self, a, head_dim): return _lib.ref_rope(self.h, a, head_dim)
    def rms_norm(self, x, w, eps): return _lib.ref_rms_norm(self.h, x, w, float(eps))
    def repeat_kv(self, x, repeats): return _lib.ref_repeat_kv(self.h, x, repeats)
    def sum(self, a, dim): return _lib.ref_sum(self.h, a, dim)
    def max(self, a, dim): return _lib.ref_max(self.h, a, dim)
    def transpose(self, a, d0, d1): return _lib.ref_transpose(self.h, a, d0, d1)
    def backward(self, loss): _lib.ref_backward(self.h, loss)

    def flash_attention(self, q, k, v, scale, causal):
        return _lib.ref_flash_attention(self.h, q, k, v, float(scale), int(causal))

    def reshape(self, a, shape):
        sh, rank = _shape(tuple(shape))
        return _lib.ref_reshape(self.h, a, sh, rank)

    def cross_entropy(self, logits, targets):
        t = np.ascontiguousarray(targets, dtype=np.int64)
        return _lib.ref_cross_entropy(self.h, logits, ip(t))

    def cross_entropy_masked(self, logits, targets):
        t = np.ascontiguousarray(targets, dtype=np.int64)
        return _lib.ref_cross_entropy_masked(self.h, logits, ip(t))

    def gqa_forward(self, heads, kv_heads, head_dim, wq, wk, wv, wo, x, causal=True):
        return _lib.ref_gqa_forward(self.h, heads, kv_heads, head_dim, wq, wk, wv, wo, x, int(causal))


def attention_chain(q, k, v, do, scale, causal=True):
    """q, do: [B,S,Hq,hd]; k, v: [B,S,Hkv,hd].  The reference's training chain
    (src/nn/attention.rs:319-378): transpose_0213, repeat_kv, bmm(q,k^T), mul(scale), add(mask),
    softmax, bmm(p,v), transpose back.  Returns O, dQ, dK, dV in the input layouts."""
    B, S, Hq, hd = q.shape
    Hkv = k.shape[2]
    g = Graph()
    qi, ki, vi = g.alloc(q.shape, q), g.alloc(k.shape, k), g.alloc(v.shape, v)
    qt, kt, vt = g.transpose_0213(qi), g.transpose_0213(ki), g.transpose_0213(vi)
    kr, vr = g.repeat_kv(kt, Hq // Hkv), g.repeat_kv(vt, Hq // Hkv)
    for t in (qt, kr, vr):
        g.reinterpret_shape(t, (B * Hq, S, hd))
    sc = g.bmm(qt, kr, True)
    sc = g.mul_const(sc, g.alloc((B * Hq, S, S), np.full((B * Hq, S, S), scale, np.float32)))
    if causal:
        sc = g.add(sc, g.alloc((1, S, S), np.triu(np.full((S, S), -1e20, np.float32), 1)))
    ctx_ = g.bmm(g.softmax(sc), vr, False)
    g.reinterpret_shape(ctx_, (B, Hq, S, hd))
    o = g.transpose_0213(ctx_)
    seed = g.alloc(do.shape, do)
    g.backward(g.sum(g.sum(g.sum(g.sum(g.mul(o, seed), 3), 2), 1), 0))
    return g.data(o), g.grad(qi), g.grad(ki), g.grad(vi)


class TransformerLM:
    """Mirror of src/nn/transformer.rs TransformerLM over the C oracle."""

    def __init__(self, g, vocab, hidden, heads, kv_heads, ffn, layers, tie):
        self.g = g
        self.cfg = dict(vocab=vocab, hidden=hidden, heads=heads, kv_heads=kv_heads, ffn=ffn, layers=layers, tie=tie)
        self.h = _lib.ref_lm_new(g.h, vocab, hidden, heads, kv_heads, ffn, layers, int(tie))
        buf = (C.c_int * (layers * 9 + 3))()
        n = _lib.ref_lm_params(self.h, buf)
        self._params = list(buf[:n])

    def __del__(self):
        if getattr(self, "h", None):
            _lib.ref_lm_free(self.h)
            self.h = None

    def params(self):
        return list(self._params)

    def forward(self, x_id):
        return _lib.ref_lm_forward(self.g.h, self.h, x_id)

    def micro_step(self, ids, targets):
        """ids [mb, seq] (any int/float dtype), targets [mb*seq] int64. Returns the loss."""
        ids = _f32(ids)
        mb, seq = ids.shape
        t = np.ascontiguousarray(targets, dtype=np.int64).reshape(-1)
        return float(_lib.ref_lm_micro_step(self.g.h, self.h, fp(ids), ip(t), mb, seq))


class AdamW:
    """Mirror of src/nn/optim.rs AdamW over the C oracle."""

    def __init__(self, g, params, lr):
        self.g = g
        self.params = list(params)
        arr = (C.c_int * len(params))(*params)
        self.h = _lib.ref_adamw_new(g.h, arr, len(params), float(lr))

    def __del__(self):
        if getattr(self, "h", None):
            _lib.ref_adamw_free(self.h)
            self.h = None

    def config(self, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, grad_clip_norm=0.0):
        _lib.ref_adamw_config(self.h, lr, beta1, beta2, eps, weight_decay, grad_clip_norm)

    def zero_grad(self):
        _lib.ref_adamw_zero_grad(self.h, self.g.h)

    def clip_grad_norm(self, max_norm):
        coef = C.c_float()
        norm = _lib.ref_adamw_clip_grad_norm(self.h, self.g.h, float(max_norm), C.byref(coef))
        return norm, coef.value

    def step(self):
        _lib.ref_adamw_step(self.h, self.g.h)

    def moments(self, i):
        n = _lib.ref_numel(self.g.h, self.params[i])
        m = np.ctypeslib.as_array(_lib.ref_adamw_m(self.h, i), (n,)).copy()
        v = np.ctypeslib.as_array(_lib.ref_adamw_v(self.h, i), (n,)).copy()
        return m, v
