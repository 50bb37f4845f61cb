"""ctypes mirror of include/eisen_graph.h: Graph, TransformerLM, AdamW with the reference's method names."""
import ctypes as C
import weakref

import numpy as np

from .hip import Context
from .lib import EisenHipError

FP32, BF16_MIXED = 0, 1
_sz, _f, _i, _vp = C.c_size_t, C.c_float, C.c_int, C.c_void_p
_f32p = C.POINTER(C.c_float)


def _shape(shape):
    shape = tuple(int(s) for s in shape)
    return (C.c_size_t * max(len(shape), 1))(*shape), len(shape)


def _fp(a):
    return a.ctypes.data_as(_f32p)


class Graph:
    """`Graph::new(Device::Gpu(..))` (src/graph/mod.rs:152-307) over the C++ host layer."""

    def __init__(self, ctx: Context, precision=FP32):
        self.ctx = ctx
        self.lib = ctx.lib
        self.lib.eisen_graph_last_error.restype = C.c_char_p
        self.lib.eisen_cosine_lr.restype = C.c_float
        h = _vp()
        rc = self.lib.eisen_graph_new(ctx.h, int(precision), C.byref(h))
        if rc:
            raise EisenHipError("eisen_graph_new", rc, "could not create the graph")
        self.h = h
        self.precision = precision
        self._children = []      # modules and optimisers hold device memory of this graph
        ctx._children.append(weakref.ref(self))

    def close(self):
        if getattr(self, "h", None):
            for ref in self._children:
                child = ref()
                if child is not None:
                    child.close()
            if getattr(self.ctx, "h", None):
                self.lib.eisen_graph_free(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def _call(self, name, *args):
        rc = getattr(self.lib, name)(self.h, *args)
        if rc:
            raise EisenHipError(name, rc, self.lib.eisen_graph_last_error(self.h).decode())

    def _op(self, name, *args):
        out = _sz()
        self._call(name, *args, C.byref(out))
        return out.value

    # ---- runtime ----------------------------------------------------------------------
    def alloc(self, shape, data):
        d = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        sh, rank = _shape(shape)
        return self._op("eisen_graph_alloc", sh, _i(rank), _fp(d))

    def alloc_pooled(self, shape):
        sh, rank = _shape(shape)
        return self._op("eisen_graph_alloc_pooled", sh, _i(rank))

    def load_tensor_data(self, tid, data):
        d = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        self._call("eisen_graph_load_tensor_data", _sz(tid), _fp(d), _sz(d.size))

    def input(self, data):
        """An activation-typed tensor holding `data` (alloc_pooled + load_tensor_data, train_llm.rs:433-435)."""
        data = np.asarray(data, dtype=np.float32)
        tid = self.alloc_pooled(data.shape)
        self.load_tensor_data(tid, data)
        return tid

    def mark_params(self): self._call("eisen_graph_mark_params")
    def clear_activations(self): self._call("eisen_graph_clear_activations")
    def synchronize(self): self._call("eisen_graph_synchronize")
    def set_no_grad(self, v): self._call("eisen_graph_set_no_grad", _i(int(v)))
    def restore_save_point(self, sp): self._call("eisen_graph_restore_save_point", _sz(sp))

    def set_weight_gradient_window(self, backward_passes): self._call("eisen_graph_set_weight_gradient_window", _sz(backward_passes))
    def set_weight_gradients_beside(self, on): self._call("eisen_graph_set_weight_gradients_beside", _i(int(on)))
    def flush_weight_gradients(self): self._call("eisen_graph_flush_weight_gradients")

    def restore_save_point_keep(self, sp, keep):
        out = _sz()
        self._call("eisen_graph_restore_save_point_keep", _sz(sp), _sz(keep), C.byref(out))
        return out.value

    def mark_save_point(self):
        out = _sz()
        self._call("eisen_graph_mark_save_point", C.byref(out))
        return out.value

    def _count(self, name):
        out = _sz()
        self._call(name, C.byref(out))
        return out.value

    def num_tensors(self): return self._count("eisen_graph_num_tensors")
    def num_params(self): return self._count("eisen_graph_num_params")
    def tape_len(self): return self._count("eisen_graph_tape_len")

    def shape(self, tid):
        sh = (C.c_size_t * 8)()
        rank = _i()
        self._call("eisen_graph_tensor_shape", _sz(tid), sh, C.byref(rank))
        return tuple(sh[:rank.value])

    def reinterpret_shape(self, tid, shape):
        sh, rank = _shape(shape)
        self._call("eisen_graph_reinterpret_shape", _sz(tid), sh, _i(rank))

    def sync_to_cpu(self, tid):
        shape = self.shape(tid)
        out = np.empty(shape, np.float32)
        self._call("eisen_graph_sync_to_cpu", _sz(tid), _fp(out), _sz(out.size))
        return out

    def sync_grad_to_cpu(self, tid):
        shape = self.shape(tid)
        out = np.empty(shape, np.float32)
        self._call("eisen_graph_sync_grad_to_cpu", _sz(tid), _fp(out), _sz(out.size))
        return out

    def sync_compute_copy_to_cpu(self, tid):
        """The values the kernels read for this tensor (a mixed-mode parameter's bf16 copy), widened to f32."""
        out = np.empty(self.shape(tid), np.float32)
        self._call("eisen_graph_sync_compute_copy_to_cpu", _sz(tid), _fp(out), _sz(out.size))
        return out

    # ---- ops --------------------------------------------------------------------------
    def add(self, a, b): return self._op("eisen_graph_add", _sz(a), _sz(b))
    def mul(self, a, b): return self._op("eisen_graph_mul", _sz(a), _sz(b))
    def silu(self, a): return self._op("eisen_graph_silu", _sz(a))
    def swiglu(self, gate, up): return self._op("eisen_graph_swiglu", _sz(gate), _sz(up))
    def matmul(self, a, b): return self._op("eisen_graph_matmul", _sz(a), _sz(b))
    def matmul_trans_b(self, a, b): return self._op("eisen_graph_matmul_trans_b", _sz(a), _sz(b))
    def bmm(self, a, b, trans_b): return self._op("eisen_graph_bmm", _sz(a), _sz(b), _i(int(trans_b)))
    def softmax(self, a): return self._op("eisen_graph_softmax", _sz(a))
    def transpose_0213(self, a): return self._op("eisen_graph_transpose_0213", _sz(a))
    def gather(self, w, idx): return self._op("eisen_graph_gather", _sz(w), _sz(idx))
    def rope(self, a, head_dim): return self._op("eisen_graph_rope", _sz(a), _sz(head_dim))
    def rms_norm(self, x, w, eps): return self._op("eisen_graph_rms_norm", _sz(x), _sz(w), _f(eps))
    def repeat_kv(self, x, repeats): return self._op("eisen_graph_repeat_kv", _sz(x), _sz(repeats))

    def reshape(self, a, shape):
        sh, rank = _shape(shape)
        return self._op("eisen_graph_reshape", _sz(a), sh, _i(rank))

    def _targets(self, targets):
        t = np.ascontiguousarray(targets, dtype=np.int64).reshape(-1)
        return t, t.ctypes.data_as(C.POINTER(C.c_int64))

    def cross_entropy(self, logits, targets):
        t, p = self._targets(targets)
        return self._op("eisen_graph_cross_entropy", _sz(logits), p, _sz(t.size))

    def cross_entropy_masked(self, logits, targets):
        t, p = self._targets(targets)
        return self._op("eisen_graph_cross_entropy_masked", _sz(logits), p, _sz(t.size))

    def flash_attention(self, q, k, v, scale, causal):
        return self._op("eisen_graph_flash_attention", _sz(q), _sz(k), _sz(v), _f(scale), _i(int(causal)))

    def attention_gqa(self, q, k, v, heads, kv_heads, scale, causal=True):
        return self._op("eisen_graph_attention_gqa", _sz(q), _sz(k), _sz(v), _sz(heads), _sz(kv_heads), _f(scale), _i(int(causal)))

    def backward(self, loss): self._call("eisen_graph_backward", _sz(loss))

    def cosine_lr(self, lr_max, lr_min, warmup, total, step):
        return self.lib.eisen_cosine_lr(_f(lr_max), _f(lr_min), _sz(warmup), _sz(total), _sz(step))


class TransformerLM:
    """src/nn/transformer.rs TransformerLM."""

    def __init__(self, g: Graph, vocab, hidden, heads, kv_heads, ffn, layers, tie):
        self.g = g
        self.cfg = dict(vocab=vocab, hidden=hidden, heads=heads, kv_heads=kv_heads, ffn=ffn, layers=layers, tie=tie)
        h = _vp()
        g._call("eisen_lm_new", _sz(vocab), _sz(hidden), _sz(heads), _sz(kv_heads), _sz(ffn), _sz(layers), _i(int(tie)), C.byref(h))
        self.h = h
        g._children.append(weakref.ref(self))

    def close(self):
        if getattr(self, "h", None):
            if getattr(self.g, "h", None):
                self.g.lib.eisen_lm_free(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def _check(self, name, rc):
        if rc:
            raise EisenHipError(name, rc, self.g.lib.eisen_graph_last_error(self.g.h).decode())

    def params(self):
        n = _sz()
        self._check("eisen_lm_params", self.g.lib.eisen_lm_params(self.h, None, _sz(0), C.byref(n)))
        ids = (C.c_size_t * n.value)()
        self._check("eisen_lm_params", self.g.lib.eisen_lm_params(self.h, ids, _sz(n.value), C.byref(n)))
        return list(ids)

    def set_fused(self, fused):
        self._check("eisen_lm_set_fused", self.g.lib.eisen_lm_set_fused(self.h, _i(int(fused))))

    def set_checkpointing(self, on):
        self._check("eisen_lm_set_checkpointing", self.g.lib.eisen_lm_set_checkpointing(self.h, _i(int(on))))

    def forward(self, x_id):
        return self.g._op("eisen_lm_forward", self.h, _sz(x_id))

    def micro_step(self, ids, targets, want_loss=True):
        ids = np.ascontiguousarray(ids, dtype=np.float32)
        mb, seq = ids.shape
        t = np.ascontiguousarray(targets, dtype=np.int64).reshape(-1)
        loss = _f()
        self.g._call("eisen_lm_micro_step", self.h, _fp(ids), t.ctypes.data_as(C.POINTER(C.c_int64)), _sz(mb), _sz(seq),
                     C.byref(loss) if want_loss else None)
        return loss.value if want_loss else None


class AdamW:
    """src/nn/optim.rs AdamW."""

    def __init__(self, g: Graph, params, lr):
        self.g = g
        self.params = list(params)
        arr = (C.c_size_t * len(self.params))(*self.params)
        h = _vp()
        g._call("eisen_adamw_new", arr, _sz(len(self.params)), _f(lr), C.byref(h))
        self.h = h
        g._children.append(weakref.ref(self))

    def close(self):
        if getattr(self, "h", None):
            if getattr(self.g, "h", None):
                self.g.lib.eisen_adamw_free(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def _call(self, name, *args):
        rc = getattr(self.g.lib, name)(self.h, *args)
        if rc:
            raise EisenHipError(name, rc, self.g.lib.eisen_graph_last_error(self.g.h).decode())

    def config(self, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, grad_clip_norm=0.0):
        self._call("eisen_adamw_config", _f(lr), _f(beta1), _f(beta2), _f(eps), _f(weight_decay), _f(grad_clip_norm))

    def init_moments(self): self._call("eisen_adamw_init_moments")
    def zero_grad(self): self._call("eisen_adamw_zero_grad")
    def step(self): self._call("eisen_adamw_step")

    def clip_grad_norm(self, max_norm):
        n, c = _f(), _f()
        self._call("eisen_adamw_clip_grad_norm", _f(max_norm), C.byref(n), C.byref(c))
        return n.value, c.value

    def last_grad_norm(self):
        n, c = _f(), _f()
        self._call("eisen_adamw_last_grad_norm", C.byref(n), C.byref(c))
        return n.value, c.value

    def moments(self, i):
        n = int(np.prod(self.g.shape(self.params[i]), dtype=np.int64))
        m, v = np.empty(n, np.float32), np.empty(n, np.float32)
        self._call("eisen_adamw_moments_to_cpu", _sz(i), _fp(m), _fp(v), _sz(n))
        return m, v
