"""ctypes mirror of include/eisen_hip.h: a Context object whose methods are the C entry points.

Buffers are raw device pointers owned by the library's stream-ordered pool; numpy is the
host side.  bf16 is carried on the host as uint16 bit patterns (round-to-nearest-even).
"""
import ctypes as C

import numpy as np

from .lib import HSACO_PATH, EisenHipError, load_library

F32, BF16 = 0, 1
IGNORE_INDEX = -1
_vp, _sz, _f, _i = C.c_void_p, C.c_size_t, C.c_float, C.c_int


def f32_to_bf16_bits(x):
    """float32 array -> uint16 bf16 bit patterns, round-to-nearest-even (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = ((u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, np.uint16(0x7FC0), rounded)
    return rounded


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(x):
    """float32 -> nearest bf16 value, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x)).reshape(np.shape(x))


class ParamSlot(C.Structure):
    _fields_ = [("w", _vp), ("g", _vp), ("m", _vp), ("v", _vp), ("w_bf16", _vp), ("n", _sz)]


class ProfEntry(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("ms", C.c_double), ("work", C.c_double), ("launches", C.c_ulonglong), ("work_is_flops", C.c_int)]


class Buffer:
    """A device allocation from the context's pool."""

    def __init__(self, ctx, ptr, nbytes):
        self.ctx, self.ptr, self.nbytes = ctx, ptr, nbytes

    def free(self):
        if self.ptr:
            self.ctx._call("eisen_hip_free", _vp(self.ptr))
            self.ptr = 0

    def __int__(self):
        return self.ptr


def _ptr(b):
    if b is None:
        return _vp(0)
    return _vp(b.ptr if isinstance(b, Buffer) else int(b))


class Context:
    def __init__(self, device=0):
        self.lib = load_library()
        self.lib.eisen_hip_last_error.restype = C.c_char_p
        self.lib.eisen_hip_stream.restype = _vp
        h = _vp()
        rc = self.lib.eisen_hip_init(int(device), C.byref(h))
        if rc != 0:
            raise EisenHipError("eisen_hip_init", rc, "no usable HIP device" if rc > 0 else "bad device index")
        self.h = h
        self._children = []     # weak references to Graph objects created on this context

    def close(self):
        if getattr(self, "h", None):
            for ref in getattr(self, "_children", []):
                child = ref()
                if child is not None:
                    child.close()
            self.lib.eisen_hip_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def _call(self, name, *args):
        rc = getattr(self.lib, name)(self.h, *args)
        if rc != 0:
            raise EisenHipError(name, rc, self.lib.eisen_hip_last_error(self.h).decode())

    # ---- memory -----------------------------------------------------------------------
    def malloc(self, nbytes, zero=False):
        p = _vp()
        self._call("eisen_hip_malloc_zeroed" if zero else "eisen_hip_malloc", _sz(nbytes), C.byref(p))
        return Buffer(self, p.value, nbytes)

    def upload(self, arr, dtype=None):
        """numpy -> device.  dtype BF16 converts a float array to bf16 bits first."""
        arr = np.asarray(arr)
        if dtype == BF16:
            arr = f32_to_bf16_bits(arr)
        elif dtype == F32:
            arr = np.ascontiguousarray(arr, dtype=np.float32)
        arr = np.ascontiguousarray(arr)
        buf = self.malloc(max(arr.nbytes, 4))
        if arr.nbytes:
            self._call("eisen_hip_htod", _vp(buf.ptr), arr.ctypes.data_as(_vp), _sz(arr.nbytes))
        return buf

    def download(self, buf, shape, dtype=F32):
        """device -> numpy float32 (dtype F32/BF16) or the given numpy dtype."""
        shape = tuple(int(s) for s in np.atleast_1d(shape)) if not isinstance(shape, tuple) else shape
        if dtype == BF16:
            out = np.empty(shape, np.uint16)
        elif dtype == F32:
            out = np.empty(shape, np.float32)
        else:
            out = np.empty(shape, dtype)
        if out.nbytes:
            self._call("eisen_hip_dtoh", out.ctypes.data_as(_vp), _ptr(buf), _sz(out.nbytes))
        return bf16_bits_to_f32(out).reshape(shape) if dtype == BF16 else out

    def dtoh_begin(self, buf, nbytes):
        """Queue a device-to-host copy; returns a ticket for dtoh_finish."""
        t = C.c_int(-1)
        self._call("eisen_hip_dtoh_begin", _ptr(buf), _sz(nbytes), C.byref(t))
        return t.value

    def dtoh_finish(self, ticket, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        self._call("eisen_hip_dtoh_finish", _i(ticket), out.ctypes.data_as(_vp), _sz(out.nbytes))
        return out

    def sync(self):
        self._call("eisen_hip_stream_sync")

    def mem_info(self):
        f, t = _sz(), _sz()
        self._call("eisen_hip_mem_info", C.byref(f), C.byref(t))
        return f.value, t.value

    def pool_stats(self):
        a, b = _sz(), _sz()
        self._call("eisen_hip_pool_stats", C.byref(a), C.byref(b))
        return a.value, b.value

    def driver_allocs(self):
        n = _sz()
        self._call("eisen_hip_driver_allocs", C.byref(n))
        return n.value

    def pool_peak(self, reset=False):
        a = _sz()
        self._call("eisen_hip_pool_peak", C.byref(a), _i(int(reset)))
        return a.value

    def pool_trim(self):
        self._call("eisen_hip_pool_trim")

    def memset_zero(self, buf, nbytes):
        self._call("eisen_hip_memset_zero", _ptr(buf), _sz(nbytes))

    def dtod(self, dst, src, nbytes):
        self._call("eisen_hip_dtod", _ptr(dst), _ptr(src), _sz(nbytes))

    def timer_start(self):
        self._call("eisen_hip_timer_start")

    def timer_stop(self):
        ms = _f()
        self._call("eisen_hip_timer_stop", C.byref(ms))
        return ms.value

    def profile_start(self):
        """Bracket every instrumented kernel launch with HIP events on the context's stream."""
        self._call("eisen_hip_profile_start")

    def profile_stop(self):
        """-> {kernel family: dict(ms, launches, work, unit)}; synchronises."""
        arr = (ProfEntry * 64)()
        n = _sz()
        self._call("eisen_hip_profile_stop", arr, _sz(64), C.byref(n))
        out = {}
        for e in arr[:min(n.value, 64)]:
            out[e.name.decode()] = dict(ms=e.ms, launches=int(e.launches), work=e.work, unit="flop" if e.work_is_flops else "byte")
        return out

    def mfma_ceiling(self, lds_reads_per_16_mfma=0, iters=20000, random_operands=False):
        """TFLOP/s of a loop of nothing but bf16 MFMAs on every CU (operands in registers, or re-read from LDS); with
        random_operands the operands' bits change from MFMA to MFMA as real data's do, which lowers the clock the part holds."""
        out = C.c_double()
        self._call("eisen_hip_mfma_ceiling_random" if random_operands else "eisen_hip_mfma_ceiling", _i(lds_reads_per_16_mfma), _i(iters), C.byref(out))
        return out.value

    # ---- by-name launch ---------------------------------------------------------------
    def module_load(self, path=HSACO_PATH):
        image = open(path, "rb").read()
        self._keep = getattr(self, "_keep", []) + [image]
        m = _vp()
        self._call("eisen_hip_module_load", C.c_char_p(image), _sz(len(image)), C.byref(m))
        return m

    def get_function(self, module, name):
        f = _vp()
        self._call("eisen_hip_get_function", module, C.c_char_p(name.encode()), C.byref(f))
        return f

    def launch(self, fn, grid, block, args, shared=0):
        """args: list of ctypes values, pushed positionally like cudarc's launch_builder."""
        g = (C.c_uint * 3)(*grid)
        b = (C.c_uint * 3)(*block)
        arr = (_vp * len(args))(*[C.cast(C.pointer(a), _vp) for a in args])
        self._call("eisen_hip_launch", fn, g, b, C.c_uint(shared), arr)

    def module_unload(self, module):
        self._call("eisen_hip_module_unload", module)

    # ---- elementwise ------------------------------------------------------------------
    def fill(self, dst, dtype, value, n): self._call("eisen_hip_fill", _ptr(dst), _i(dtype), _f(value), _sz(n))
    def scale(self, dst, dtype, factor, n): self._call("eisen_hip_scale", _ptr(dst), _i(dtype), _f(factor), _sz(n))
    def scale_by_device_scalar(self, dst, dtype, factor_dev, n): self._call("eisen_hip_scale_by_device_scalar", _ptr(dst), _i(dtype), _ptr(factor_dev), _sz(n))
    def cast(self, src, src_dtype, dst, dst_dtype, n): self._call("eisen_hip_cast", _ptr(src), _i(src_dtype), _ptr(dst), _i(dst_dtype), _sz(n))
    def accumulate(self, dst, src, dtype, n, accumulate): self._call("eisen_hip_accumulate", _ptr(dst), _ptr(src), _i(dtype), _sz(n), _i(accumulate))
    def add(self, a, b, out, dtype, n): self._call("eisen_hip_add", _ptr(a), _ptr(b), _ptr(out), _i(dtype), _sz(n))
    def mul(self, a, b, out, dtype, n): self._call("eisen_hip_mul", _ptr(a), _ptr(b), _ptr(out), _i(dtype), _sz(n))

    @staticmethod
    def _szarr(v):
        return (C.c_size_t * len(v))(*[int(x) for x in v])

    def add_bcast(self, a, b, out, dtype, out_shape, a_strides, b_strides):
        self._call("eisen_hip_add_bcast", _ptr(a), _ptr(b), _ptr(out), _i(dtype), _i(len(out_shape)), self._szarr(out_shape), self._szarr(a_strides), self._szarr(b_strides))

    def mul_bcast(self, a, b, out, dtype, out_shape, a_strides, b_strides):
        self._call("eisen_hip_mul_bcast", _ptr(a), _ptr(b), _ptr(out), _i(dtype), _i(len(out_shape)), self._szarr(out_shape), self._szarr(a_strides), self._szarr(b_strides))

    def bcast_backward(self, dst, go, other, dtype, out_shape, dst_strides, other_strides, dst_numel, accumulate):
        self._call("eisen_hip_bcast_backward", _ptr(dst), _ptr(go), _ptr(other), _i(dtype), _i(len(out_shape)), self._szarr(out_shape),
                   self._szarr(dst_strides), self._szarr(other_strides) if other_strides is not None else None, _sz(dst_numel), _i(accumulate))

    def mul_backward(self, a, b, go, ga, gb, dtype, n, acc_a=0, acc_b=0):
        self._call("eisen_hip_mul_backward", _ptr(a), _ptr(b), _ptr(go), _ptr(ga), _ptr(gb), _i(dtype), _sz(n), _i(acc_a), _i(acc_b))

    def silu(self, x, out, dtype, n): self._call("eisen_hip_silu", _ptr(x), _ptr(out), _i(dtype), _sz(n))
    def silu_backward(self, x, go, gx, dtype, n, accumulate=0): self._call("eisen_hip_silu_backward", _ptr(x), _ptr(go), _ptr(gx), _i(dtype), _sz(n), _i(accumulate))
    def swiglu(self, gate, up, out, dtype, n): self._call("eisen_hip_swiglu", _ptr(gate), _ptr(up), _ptr(out), _i(dtype), _sz(n))

    def swiglu_backward(self, gate, up, go, dgate, dup, dtype, n, acc_gate=0, acc_up=0):
        self._call("eisen_hip_swiglu_backward", _ptr(gate), _ptr(up), _ptr(go), _ptr(dgate), _ptr(dup), _i(dtype), _sz(n), _i(acc_gate), _i(acc_up))

    # ---- norm / rope / layout ---------------------------------------------------------
    def rms_norm(self, x, w, out, rrms, dtype, rows, dim, eps):
        self._call("eisen_hip_rms_norm", _ptr(x), _ptr(w), _ptr(out), _ptr(rrms), _i(dtype), _sz(rows), _sz(dim), _f(eps))

    def rms_norm_backward(self, x, w, rrms, go, gx, gw, dtype, rows, dim, accumulate_x=0):
        self._call("eisen_hip_rms_norm_backward", _ptr(x), _ptr(w), _ptr(rrms), _ptr(go), _ptr(gx), _ptr(gw), _i(dtype), _sz(rows), _sz(dim), _i(accumulate_x))

    RMS_NORM_PARTIAL_ROWS = 256

    def rms_norm_backward_partial(self, x, w, rrms, go, gx, partial, dtype, rows, dim, accumulate_x=0):
        """dx, and the gain gradient as rows of `partial` ([RMS_NORM_PARTIAL_ROWS, dim] f32); returns the rows written."""
        n = C.c_size_t(0)
        self._call("eisen_hip_rms_norm_backward_partial", _ptr(x), _ptr(w), _ptr(rrms), _ptr(go), _ptr(gx), _ptr(partial), C.byref(n), _i(dtype),
                   _sz(rows), _sz(dim), _i(accumulate_x))
        return n.value

    def rms_norm_backward_partial_add(self, x, w, rrms, go, gx_in, gx, partial, dtype, rows, dim):
        """rms_norm_backward_partial with gx = gx_in + dx (gx_in may be gx)."""
        n = C.c_size_t(0)
        self._call("eisen_hip_rms_norm_backward_partial_add", _ptr(x), _ptr(w), _ptr(rrms), _ptr(go), _ptr(gx_in), _ptr(gx), _ptr(partial), C.byref(n),
                   _i(dtype), _sz(rows), _sz(dim))
        return n.value

    def rms_norm_dw_finish(self, partials, gws, nrows, dim, assign=None):
        """gw_i (+)= column sums of the first nrows_i rows of partial_i, all in one launch; assign[i]: overwrite gw_i."""
        n = len(partials)
        pp = (_vp * n)(*[_ptr(p) for p in partials])
        pg = (_vp * n)(*[_ptr(g) for g in gws])
        pn = (C.c_size_t * n)(*nrows)
        pa = None if assign is None else (C.c_int * n)(*[int(a) for a in assign])
        self._call("eisen_hip_rms_norm_dw_finish", _sz(n), pp, pg, pn, _sz(dim), pa)

    def rope(self, x, out, dtype, batch, seq, hidden, head_dim):
        self._call("eisen_hip_rope", _ptr(x), _ptr(out), _i(dtype), _sz(batch), _sz(seq), _sz(hidden), _sz(head_dim))

    def rope_pair(self, q, q_out, hidden_q, k, k_out, hidden_k, dtype, batch, seq, head_dim):
        self._call("eisen_hip_rope_pair", _ptr(q), _ptr(q_out), _sz(hidden_q), _ptr(k), _ptr(k_out), _sz(hidden_k), _i(dtype), _sz(batch), _sz(seq), _sz(head_dim))

    def gemm_rope(self, A, B, Cm, dtype, batch, M, N, K, stride_b, stride_c, rope_members, seq, head_dim):
        self._call("eisen_hip_gemm_rope", _ptr(A), _ptr(B), _ptr(Cm), _i(dtype), _sz(batch), _sz(M), _sz(N), _sz(K), C.c_longlong(stride_b),
                   C.c_longlong(stride_c), _sz(rope_members), _sz(seq), _sz(head_dim))

    def rope_backward(self, go, gx, dtype, batch, seq, hidden, head_dim, accumulate=0):
        self._call("eisen_hip_rope_backward", _ptr(go), _ptr(gx), _i(dtype), _sz(batch), _sz(seq), _sz(hidden), _sz(head_dim), _i(accumulate))

    def transpose_0213(self, inp, out, dtype, b, s, h, d, accumulate=0):
        self._call("eisen_hip_transpose_0213", _ptr(inp), _ptr(out), _i(dtype), _sz(b), _sz(s), _sz(h), _sz(d), _i(accumulate))

    def repeat_kv(self, inp, out, dtype, batch, kv_heads, seq, head_dim, repeats):
        self._call("eisen_hip_repeat_kv", _ptr(inp), _ptr(out), _i(dtype), _sz(batch), _sz(kv_heads), _sz(seq), _sz(head_dim), _sz(repeats))

    def repeat_kv_backward(self, go, gin, dtype, batch, kv_heads, seq, head_dim, repeats, accumulate=0):
        self._call("eisen_hip_repeat_kv_backward", _ptr(go), _ptr(gin), _i(dtype), _sz(batch), _sz(kv_heads), _sz(seq), _sz(head_dim), _sz(repeats), _i(accumulate))

    def softmax(self, x, out, dtype, rows, n): self._call("eisen_hip_softmax", _ptr(x), _ptr(out), _i(dtype), _sz(rows), _sz(n))

    def softmax_backward(self, out, go, gx, dtype, rows, n, accumulate=0):
        self._call("eisen_hip_softmax_backward", _ptr(out), _ptr(go), _ptr(gx), _i(dtype), _sz(rows), _sz(n), _i(accumulate))

    # ---- contractions -----------------------------------------------------------------
    def gemm(self, A, B, Cbuf, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, accumulate=0):
        self._call("eisen_hip_gemm", _ptr(A), _ptr(B), _ptr(Cbuf), _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(M), _sz(N), _sz(K), _i(accumulate))

    def bmm(self, A, B, Cbuf, dtype_ab, dtype_c, trans_a, trans_b, batch, M, N, K, accumulate=0):
        self._call("eisen_hip_bmm", _ptr(A), _ptr(B), _ptr(Cbuf), _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(batch), _sz(M), _sz(N), _sz(K), _i(accumulate))

    def gemm_strided_batched(self, A, B, Cbuf, dtype_ab, dtype_c, trans_a, trans_b, batch, M, N, K, stride_a, stride_b, stride_c, accumulate=0):
        """Batch strides in elements; 0 shares the operand, negative walks backwards."""
        self._call("eisen_hip_gemm_strided_batched", _ptr(A), _ptr(B), _ptr(Cbuf), _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(batch),
                   _sz(M), _sz(N), _sz(K), C.c_longlong(stride_a), C.c_longlong(stride_b), C.c_longlong(stride_c), _i(accumulate))

    def side_begin(self): self._call("eisen_hip_side_begin")
    def side_end(self): self._call("eisen_hip_side_end")
    def side_wait(self): self._call("eisen_hip_side_wait")

    def gemm_residual(self, A, B, R, Cbuf, dtype_ab, dtype_c, trans_a, trans_b, M, N, K):
        """C = R + op(A) op(B)."""
        self._call("eisen_hip_gemm_residual", _ptr(A), _ptr(B), _ptr(R), _ptr(Cbuf), _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(M), _sz(N), _sz(K))

    def gemm_grouped(self, As, Bs, Cs, Ns, dtype_ab, dtype_c, trans_a, trans_b, M, K, accumulate=0):
        """C_p (+)= op(A_p) op(B_p) for up to eight products sharing M and K."""
        n = len(Ns)
        pa = (_vp * n)(*[_ptr(a) for a in As])
        pb = (_vp * n)(*[_ptr(b) for b in Bs])
        pc = (_vp * n)(*[_ptr(c) for c in Cs])
        pn = (C.c_size_t * n)(*Ns)
        self._call("eisen_hip_gemm_grouped", _sz(n), pa, pb, pc, pn, _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(M), _sz(K), _i(accumulate))

    def gemm_grouped_ksegments(self, As, Bs, Cs, Ms, Ns, seg_k, accumulate=0):
        """C_p (+)= sum_s As[p][s]^T Bs[p][s]: bf16 pieces [seg_k, M_p] and [seg_k, N_p], f32 results."""
        n, ns = len(Cs), len(As[0])
        pa = (_vp * (n * ns))(*[_ptr(a) for row in As for a in row])
        pb = (_vp * (n * ns))(*[_ptr(b) for row in Bs for b in row])
        pc = (_vp * n)(*[_ptr(c) for c in Cs])
        pm = (C.c_size_t * n)(*Ms)
        pn = (C.c_size_t * n)(*Ns)
        self._call("eisen_hip_gemm_grouped_ksegments", _sz(n), _sz(ns), pa, pb, pc, pm, pn, _sz(seg_k), _i(accumulate))

    def gemm_swiglu_forward(self, X, Wg, Wu, G, U, H, dtype, M, N, K):
        """G = X Wg, U = X Wu, H = silu(G) * U."""
        self._call("eisen_hip_gemm_swiglu_forward", _ptr(X), _ptr(Wg), _ptr(Wu), _ptr(G), _ptr(U), _ptr(H), _i(dtype), _sz(M), _sz(N), _sz(K))

    def gemm_swiglu_backward(self, A, B, gate, up, dgate, dup, dtype, trans_a, trans_b, M, N, K):
        """[dgate, dup] = d(silu(gate) * up) for dH = op(A) op(B)."""
        self._call("eisen_hip_gemm_swiglu_backward", _ptr(A), _ptr(B), _ptr(gate), _ptr(up), _ptr(dgate), _ptr(dup), _i(dtype), _i(trans_a), _i(trans_b),
                   _sz(M), _sz(N), _sz(K))

    def gemm_window_meet(self, microseconds):
        """Longest wait at the meeting points of gemm_grouped_ksegments' one-launch form (0 = no meeting points)."""
        self._call("eisen_hip_gemm_window_meet", _i(microseconds))

    def gemm_ksegments(self, As, Bs, Ks, Cbuf, dtype_ab, dtype_c, trans_a, trans_b, M, N, accumulate=0):
        """C (+)= sum_s op(A_s) op(B_s) over up to three (A, B, K) segments."""
        n = len(Ks)
        pa = (_vp * n)(*[_ptr(a) for a in As])
        pb = (_vp * n)(*[_ptr(b) for b in Bs])
        ks = (C.c_size_t * n)(*Ks)
        self._call("eisen_hip_gemm_ksegments", _sz(n), pa, pb, ks, _ptr(Cbuf), _i(dtype_ab), _i(dtype_c), _i(trans_a), _i(trans_b), _sz(M), _sz(N), _i(accumulate))

    # ---- attention --------------------------------------------------------------------
    @staticmethod
    def _strides(v):
        return None if v is None else (C.c_longlong * 3)(*[int(x) for x in v])

    def attention_forward(self, q, k, v, out, lse, dtype, B, S, Hq, Hkv, hd, scale, causal=True, q_strides=None, kv_strides=None):
        self._call("eisen_hip_attention_forward", _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _i(dtype), _sz(B), _sz(S), _sz(Hq),
                   _sz(Hkv), _sz(hd), self._strides(q_strides), self._strides(kv_strides), _f(scale), _i(int(causal)))

    def attention_backward(self, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, scale, causal=True, q_strides=None,
                           kv_strides=None):
        self._call("eisen_hip_attention_backward", _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk),
                   _ptr(dv), _i(dtype), _sz(B), _sz(S), _sz(Hq), _sz(Hkv), _sz(hd), self._strides(q_strides), self._strides(kv_strides),
                   _f(scale), _i(int(causal)))

    def attention_backward_noalloc(self, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, scale, causal=True, q_strides=None,
                                   kv_strides=None):
        """attention_backward without any allocation: its scratch is a fixed device array of the library (B*Hq*S <= 2^20)."""
        self._call("eisen_hip_attention_backward_noalloc", _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk),
                   _ptr(dv), _i(dtype), _sz(B), _sz(S), _sz(Hq), _sz(Hkv), _sz(hd), self._strides(q_strides), self._strides(kv_strides),
                   _f(scale), _i(int(causal)))

    def attention_ablation(self, part):
        """Measurement only: leave one part of the backward kernels' tile loop out (0 = the real kernels)."""
        self._call("eisen_hip_attention_ablation", _i(part))

    def attention_timeline(self, stamps=None, waves=0):
        """Measurement only: the hd-64 attention kernels drop time stamps into `stamps` (3 * waves * 16 int64) until called with None."""
        self._call("eisen_hip_attention_timeline", _ptr(stamps), _sz(waves))

    def attention_tile_model(self, parts, waves_per_simd=2, iters=4000):
        """Measurement only: ns per tile and SIMD of a model of the dK/dV kernel's tile loop (parts: 1 MFMA, 3 +VALU, 7 +LDS, 8 loads, 15 all; 16 / 32 the one-pass tile with / without its dQ partial stores)."""
        out = C.c_double(0.0)
        self._call("eisen_hip_attention_tile_model", _i(parts), _i(waves_per_simd), _i(iters), C.byref(out))
        return out.value

    def attention_onepass_parts(self, rows, seq, chunk):
        """Measurement only: us of the D = rowsum(dO o O) pre-pass and of the ordered sum of causal dQ partials (key chunks of `chunk`)."""
        a, b = C.c_double(0.0), C.c_double(0.0)
        self._call("eisen_hip_attention_onepass_parts", _sz(rows), _i(seq), _i(chunk), C.byref(a), C.byref(b))
        return a.value, b.value

    def attention_rope_backward(self, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, scale, causal=True):
        """Backward for rotary-embedded q, k: dq, dk come out as gradients of the un-rotated projections."""
        self._call("eisen_hip_attention_rope_backward", _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(dq), _ptr(dk),
                   _ptr(dv), _i(dtype), _sz(B), _sz(S), _sz(Hq), _sz(Hkv), _sz(hd), _f(scale), _i(int(causal)))

    # ---- embedding --------------------------------------------------------------------
    def gather(self, weight, ids, out, dtype, n_ids, vocab, hidden):
        self._call("eisen_hip_gather", _ptr(weight), _ptr(ids), _ptr(out), _i(dtype), _sz(n_ids), _sz(vocab), _sz(hidden))

    def gather_backward(self, ids_host, go, gw, dtype, vocab, hidden):
        ids_host = np.ascontiguousarray(ids_host, dtype=np.int32).reshape(-1)
        self._call("eisen_hip_gather_backward", ids_host.ctypes.data_as(_vp), _ptr(go), _ptr(gw), _i(dtype), _sz(ids_host.size), _sz(vocab), _sz(hidden))

    def gather_backward_dev(self, ids_dev, go, gw, dtype, n_ids, vocab, hidden):
        """The scatter with int32 ids already on the device."""
        self._call("eisen_hip_gather_backward_dev", _ptr(ids_dev), _ptr(go), _ptr(gw), _i(dtype), _sz(n_ids), _sz(vocab), _sz(hidden))

    def gather_index_dev(self, ids_dev, n_ids, vocab, index):
        """The position index of the ordered scatter (3 * n_ids int32, device) from int32 ids on the device."""
        self._call("eisen_hip_gather_index_dev", _ptr(ids_dev), _sz(n_ids), _sz(vocab), _ptr(index))

    def gather_backward_indexed(self, index, go, gw, dtype, n_ids, vocab, hidden):
        """The scatter with an index built by gather_index_dev."""
        self._call("eisen_hip_gather_backward_indexed", _ptr(index), _ptr(go), _ptr(gw), _i(dtype), _sz(n_ids), _sz(vocab), _sz(hidden))

    # ---- loss -------------------------------------------------------------------------
    def cross_entropy(self, logits, targets, dlogits, row_loss, loss_out, dtype, rows, classes, normalizer, grad_scale=1.0,
                      argmax_out=None, target_logit_out=None):
        self._call("eisen_hip_cross_entropy", _ptr(logits), _ptr(targets), _ptr(dlogits), _ptr(row_loss), _ptr(loss_out),
                   _ptr(argmax_out), _ptr(target_logit_out), _i(dtype), _sz(rows), _sz(classes), _f(normalizer), _f(grad_scale))

    # ---- optimiser --------------------------------------------------------------------
    @staticmethod
    def make_slots(slots):
        """slots: list of (w, g, m, v, w_bf16 or None, n)."""
        arr = (ParamSlot * len(slots))()
        for k, (w, g, m, v, wb, n) in enumerate(slots):
            arr[k] = ParamSlot(_ptr(w), _ptr(g), _ptr(m), _ptr(v), _ptr(wb), n)
        return arr

    def adamw_step(self, slots, lr, beta1, beta2, eps, wd, bc1, bc2, grad_scale_dev=None):
        arr = self.make_slots(slots)
        self._call("eisen_hip_adamw_step", arr, _sz(len(slots)), _f(lr), _f(beta1), _f(beta2), _f(eps), _f(wd), _f(bc1), _f(bc2), _ptr(grad_scale_dev))

    def grad_norm(self, slots, max_norm, out_dev):
        arr = self.make_slots(slots)
        self._call("eisen_hip_grad_norm", arr, _sz(len(slots)), _f(max_norm), _ptr(out_dev))

    def zero_grads(self, slots):
        arr = self.make_slots(slots)
        self._call("eisen_hip_zero_grads", arr, _sz(len(slots)))
