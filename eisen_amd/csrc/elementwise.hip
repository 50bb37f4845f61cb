// Elementwise ops: fill/scale/cast/accumulate, add/mul (+broadcast), SiLU, fused SwiGLU.
// All are HBM-bound streams: 16-byte packets per lane, grid-stride, no LDS.
#include "device_utils.cuh"
#include "runtime.h"

namespace {

constexpr int kEwThreads = 256;

struct EwArgs {
    const void* in[3];
    void* out[2];
    int acc[2];
    float p0;
    const float* p_dev;  // optional device scalar
    size_t n;            // elements
};

// One op = a pure per-element function of NIN inputs giving NOUT outputs.
struct OpFill    { static constexpr int NIN = 0, NOUT = 1; static __device__ void apply(const float*, float* o, float p) { o[0] = p; } };
struct OpScale   { static constexpr int NIN = 1, NOUT = 1; static __device__ void apply(const float* i, float* o, float p) { o[0] = i[0] * p; } };
struct OpCopy    { static constexpr int NIN = 1, NOUT = 1; static __device__ void apply(const float* i, float* o, float) { o[0] = i[0]; } };
struct OpAdd     { static constexpr int NIN = 2, NOUT = 1; static __device__ void apply(const float* i, float* o, float) { o[0] = i[0] + i[1]; } };
struct OpMul     { static constexpr int NIN = 2, NOUT = 1; static __device__ void apply(const float* i, float* o, float) { o[0] = i[0] * i[1]; } };
// in: a, b, go -> ga = b*go, gb = a*go  (src/graph/ops/elementwise.rs:314-322)
struct OpMulBwd  { static constexpr int NIN = 3, NOUT = 2; static __device__ void apply(const float* i, float* o, float) { o[0] = i[1] * i[2]; o[1] = i[0] * i[2]; } };
// x*(1/(1+e^-x))  (src/graph/ops/elementwise.rs:442-447)
struct OpSilu    { static constexpr int NIN = 1, NOUT = 1; static __device__ void apply(const float* i, float* o, float) { o[0] = i[0] * (1.0f / (1.0f + __expf(-i[0]))); } };
// in: x, go -> go*(silu + sig*(1-silu))  (src/graph/ops/elementwise.rs:450-455)
struct OpSiluBwd {
    static constexpr int NIN = 2, NOUT = 1;
    static __device__ void apply(const float* i, float* o, float) {
        const float sig = 1.0f / (1.0f + __expf(-i[0]));
        const float silu = i[0] * sig;
        o[0] = i[1] * (silu + sig * (1.0f - silu));
    }
};
// in: gate, up -> silu(gate)*up
struct OpSwiglu  { static constexpr int NIN = 2, NOUT = 1; static __device__ void apply(const float* i, float* o, float) { o[0] = i[0] * (1.0f / (1.0f + __expf(-i[0]))) * i[1]; } };
// in: gate, up, go -> dgate = go*up*silu'(gate), dup = go*silu(gate)
struct OpSwigluBwd {
    static constexpr int NIN = 3, NOUT = 2;
    static __device__ void apply(const float* i, float* o, float) {
        const float sig = 1.0f / (1.0f + __expf(-i[0]));
        const float silu = i[0] * sig;
        o[0] = (i[2] * i[1]) * (silu + sig * (1.0f - silu));
        o[1] = i[2] * silu;
    }
};

template <typename TI, typename TO, typename Op, bool VEC>
__global__ __launch_bounds__(kEwThreads) void ew_kernel(EwArgs a) {
    constexpr int N = VEC ? (sizeof(TI) > sizeof(TO) ? Pack<TO>::N : Pack<TI>::N) : 1;
    // With mixed types the packet count is set by the narrower type (8 bf16); the f32 side
    // then moves two 16-byte packets per chunk.
    const size_t nchunks = a.n / N;
    const float p = a.p_dev ? a.p0 * a.p_dev[0] : a.p0;
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * blockDim.x) {
        float in[Op::NIN > 0 ? Op::NIN : 1][N];
        float out[Op::NOUT][N];
#pragma unroll
        for (int k = 0; k < Op::NIN; k++) {
            const TI* src = static_cast<const TI*>(a.in[k]) + c * N;
            if (VEC) {
#pragma unroll
                for (int h = 0; h < N / Pack<TI>::N; h++) {
                    const Pack<TI> pk = load_pack(src + h * Pack<TI>::N);
#pragma unroll
                    for (int j = 0; j < Pack<TI>::N; j++) in[k][h * Pack<TI>::N + j] = pk.get(j);
                }
            } else {
                in[k][0] = to_f32(src[0]);
            }
        }
#pragma unroll
        for (int j = 0; j < N; j++) {
            float ie[Op::NIN > 0 ? Op::NIN : 1], oe[Op::NOUT];
#pragma unroll
            for (int k = 0; k < Op::NIN; k++) ie[k] = in[k][j];
            Op::apply(ie, oe, p);
#pragma unroll
            for (int k = 0; k < Op::NOUT; k++) out[k][j] = oe[k];
        }
#pragma unroll
        for (int k = 0; k < Op::NOUT; k++) {
            if (a.out[k] == nullptr) continue;
            TO* dst = static_cast<TO*>(a.out[k]) + c * N;
            if (VEC) {
#pragma unroll
                for (int h = 0; h < N / Pack<TO>::N; h++) {
                    Pack<TO> pk;
                    if (a.acc[k]) {
                        pk = load_pack(dst + h * Pack<TO>::N);
#pragma unroll
                        for (int j = 0; j < Pack<TO>::N; j++) pk.set(j, pk.get(j) + out[k][h * Pack<TO>::N + j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < Pack<TO>::N; j++) pk.set(j, out[k][h * Pack<TO>::N + j]);
                    }
                    store_pack(dst + h * Pack<TO>::N, pk);
                }
            } else {
                dst[0] = from_f32<TO>(a.acc[k] ? to_f32(dst[0]) + out[k][0] : out[k][0]);
            }
        }
    }
}

template <typename TI, typename TO, typename Op>
int launch_ew(eisen_ctx* ctx, EwArgs a, const char* name) {
    if (a.n == 0) return 0;
    bool aligned = true;
    for (int k = 0; k < Op::NIN; k++) aligned = aligned && eisen_aligned(a.in[k], 16);
    for (int k = 0; k < Op::NOUT; k++) aligned = aligned && (a.out[k] == nullptr || eisen_aligned(a.out[k], 16));
    constexpr int N = sizeof(TI) > sizeof(TO) ? Pack<TO>::N : Pack<TI>::N;
    const size_t max_blocks = 256 * 16;
    size_t done = 0;
    if (aligned && a.n >= (size_t)N) {
        const size_t nchunks = a.n / N;
        const size_t blocks = std::min(max_blocks, eisen_ceil_div(nchunks, kEwThreads));
        EwArgs v = a;
        v.n = nchunks * N;
        ew_kernel<TI, TO, Op, true><<<dim3((unsigned)blocks), dim3(kEwThreads), 0, ctx->stream>>>(v);
        EISEN_LAUNCH_CHECK(ctx, name);
        done = nchunks * N;
    }
    if (done < a.n) {  // unaligned buffers or the last < N elements
        EwArgs t = a;
        for (int k = 0; k < Op::NIN; k++) t.in[k] = static_cast<const TI*>(a.in[k]) + done;
        for (int k = 0; k < Op::NOUT; k++)
            if (a.out[k]) t.out[k] = static_cast<TO*>(a.out[k]) + done;
        t.n = a.n - done;
        const size_t blocks = std::min(max_blocks, eisen_ceil_div(t.n, kEwThreads));
        ew_kernel<TI, TO, Op, false><<<dim3((unsigned)blocks), dim3(kEwThreads), 0, ctx->stream>>>(t);
        EISEN_LAUNCH_CHECK(ctx, name);
    }
    return 0;
}

template <typename Op>
int dispatch_ew(eisen_ctx* ctx, int dtype, EwArgs a, const char* name) {
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "%s: unknown dtype %d", name, dtype);
    for (int k = 0; k < Op::NIN; k++) EISEN_REQUIRE(ctx, a.in[k] != nullptr, EISEN_E_ARG, "%s: null input %d", name, k);
    if (dtype == EISEN_F32) return launch_ew<float, float, Op>(ctx, a, name);
    return launch_ew<bf16_t, bf16_t, Op>(ctx, a, name);
}

// ---- broadcast (rank <= 4), one thread per output element -------------------------------

struct BcastArgs {
    size_t shape[4], sa[4], sb[4];
    int rank;
    size_t n;
};

template <typename T, bool MUL>
__global__ __launch_bounds__(kEwThreads) void bcast_kernel(const T* a, const T* b, T* out, BcastArgs g) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < g.n; i += (size_t)gridDim.x * blockDim.x) {
        size_t rem = i, ia = 0, ib = 0;
#pragma unroll
        for (int d = 3; d >= 0; d--) {
            if (d < g.rank) {
                const size_t c = rem % g.shape[d];
                rem /= g.shape[d];
                ia += c * g.sa[d];
                ib += c * g.sb[d];
            }
        }
        const float x = to_f32(a[ia]), y = to_f32(b[ib]);
        out[i] = from_f32<T>(MUL ? x * y : x + y);
    }
}

// dst element -> walk every output element that maps onto it, in ascending flat order.
struct BcastBwdArgs {
    size_t shape[4], sd[4], so[4];
    int rank;
    size_t dst_numel;
};

// chunks == 1: as described.  chunks > 1 (few dst elements, long reductions: the gradient of a broadcast scalar): the walk
// of one dst element is cut into `chunks` consecutive ranges, one thread each, whose sums go to partial[e * chunks + c];
// bcast_bwd_finish_kernel adds them in ascending order.  Deterministic either way; the chunked form associates the sum
// differently from the single walk.
template <typename T, typename TD>
__global__ __launch_bounds__(kEwThreads) void bcast_bwd_kernel(TD* dst, const T* go, const T* other, BcastBwdArgs g,
                                                                int accumulate, size_t chunks, float* partial) {
    size_t fixed_shape[4], red_shape[4];
    size_t out_strides[4];
    size_t cur = 1;
    for (int d = g.rank - 1; d >= 0; d--) {
        out_strides[d] = cur;
        cur *= g.shape[d];
    }
    size_t nred = 1;
    for (int d = 0; d < g.rank; d++) {
        const bool is_red = g.sd[d] == 0 && g.shape[d] > 1;
        fixed_shape[d] = is_red ? 1 : g.shape[d];
        red_shape[d] = is_red ? g.shape[d] : 1;
        nred *= red_shape[d];
    }
    const size_t per_chunk = (nred + chunks - 1) / chunks;
    for (size_t w = (size_t)blockIdx.x * blockDim.x + threadIdx.x; w < g.dst_numel * chunks; w += (size_t)gridDim.x * blockDim.x) {
        const size_t e = w / chunks, chunk = w % chunks;
        const size_t t_lo = chunk * per_chunk, t_hi = t_lo + per_chunk < nred ? t_lo + per_chunk : nred;
        // decode e over the non-reduced dims (dst is contiguous over them in order)
        size_t rem = e, base_out = 0, base_other = 0, dst_idx = 0;
        for (int d = g.rank - 1; d >= 0; d--) {
            const size_t c = rem % fixed_shape[d];
            rem /= fixed_shape[d];
            base_out += c * out_strides[d];
            base_other += c * g.so[d];
            dst_idx += c * g.sd[d];
        }
        float acc = accumulate && chunks == 1 ? to_f32(dst[dst_idx]) : 0.f;
        for (size_t t = t_lo; t < t_hi; t++) {
            size_t r = t, io = base_out, ioth = base_other;
            for (int d = g.rank - 1; d >= 0; d--) {
                const size_t c = r % red_shape[d];
                r /= red_shape[d];
                io += c * out_strides[d];
                ioth += c * g.so[d];
            }
            const float gv = to_f32(go[io]);
            acc += other ? to_f32(other[ioth]) * gv : gv;
        }
        if (chunks == 1) dst[dst_idx] = from_f32<TD>(acc);
        else partial[w] = acc;
    }
}

template <typename T>
__global__ __launch_bounds__(kEwThreads) void bcast_bwd_finish_kernel(T* dst, const float* partial, BcastBwdArgs g, int accumulate, size_t chunks) {
    size_t fixed_shape[4];
    for (int d = 0; d < g.rank; d++) fixed_shape[d] = g.sd[d] == 0 && g.shape[d] > 1 ? 1 : g.shape[d];
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < g.dst_numel; e += (size_t)gridDim.x * blockDim.x) {
        size_t rem = e, dst_idx = 0;
        for (int d = g.rank - 1; d >= 0; d--) {
            dst_idx += (rem % fixed_shape[d]) * g.sd[d];
            rem /= fixed_shape[d];
        }
        float acc = accumulate ? to_f32(dst[dst_idx]) : 0.f;
        for (size_t c = 0; c < chunks; c++) acc += partial[e * chunks + c];
        dst[dst_idx] = from_f32<T>(acc);
    }
}

template <typename TI, typename TO>
int launch_cast(eisen_ctx* ctx, const void* src, void* dst, size_t n) {
    EwArgs a{};
    a.in[0] = src;
    a.out[0] = dst;
    a.n = n;
    return launch_ew<TI, TO, OpCopy>(ctx, a, "cast");
}

}  // namespace

extern "C" int eisen_hip_fill(eisen_ctx* ctx, void* dst, int dtype, float value, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst != nullptr, EISEN_E_ARG, "eisen_hip_fill: null dst");
    EwArgs a{};
    a.out[0] = dst;
    a.p0 = value;
    a.n = n;
    return dispatch_ew<OpFill>(ctx, dtype, a, "fill");
}

extern "C" int eisen_hip_scale(eisen_ctx* ctx, void* dst, int dtype, float factor, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst != nullptr, EISEN_E_ARG, "eisen_hip_scale: null dst");
    EwArgs a{};
    a.in[0] = dst;
    a.out[0] = dst;
    a.p0 = factor;
    a.n = n;
    return dispatch_ew<OpScale>(ctx, dtype, a, "scale");
}

extern "C" int eisen_hip_scale_by_device_scalar(eisen_ctx* ctx, void* dst, int dtype, const float* factor_device,
                                                size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst && factor_device, EISEN_E_ARG, "eisen_hip_scale_by_device_scalar: null pointer");
    EwArgs a{};
    a.in[0] = dst;
    a.out[0] = dst;
    a.p0 = 1.0f;
    a.p_dev = factor_device;
    a.n = n;
    return dispatch_ew<OpScale>(ctx, dtype, a, "scale_by_device_scalar");
}

extern "C" int eisen_hip_cast(eisen_ctx* ctx, const void* src, int src_dtype, void* dst, int dst_dtype, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, src && dst, EISEN_E_ARG, "eisen_hip_cast: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(src_dtype) && eisen_dtype_ok(dst_dtype), EISEN_E_ARG, "eisen_hip_cast: unknown dtype");
    if (src_dtype == EISEN_F32 && dst_dtype == EISEN_BF16) return launch_cast<float, bf16_t>(ctx, src, dst, n);
    if (src_dtype == EISEN_BF16 && dst_dtype == EISEN_F32) return launch_cast<bf16_t, float>(ctx, src, dst, n);
    if (src_dtype == EISEN_F32) return launch_cast<float, float>(ctx, src, dst, n);
    return launch_cast<bf16_t, bf16_t>(ctx, src, dst, n);
}

extern "C" int eisen_hip_accumulate(eisen_ctx* ctx, void* dst, const void* src, int dtype, size_t n, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst != nullptr, EISEN_E_ARG, "eisen_hip_accumulate: null dst");
    EwArgs a{};
    a.in[0] = src;
    a.out[0] = dst;
    a.acc[0] = accumulate;
    a.n = n;
    return dispatch_ew<OpCopy>(ctx, dtype, a, "accumulate");
}

extern "C" int eisen_hip_add(eisen_ctx* ctx, const void* x, const void* y, void* out, int dtype, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out != nullptr, EISEN_E_ARG, "eisen_hip_add: null out");
    EwArgs a{};
    a.in[0] = x;
    a.in[1] = y;
    a.out[0] = out;
    a.n = n;
    return dispatch_ew<OpAdd>(ctx, dtype, a, "add");
}

extern "C" int eisen_hip_mul(eisen_ctx* ctx, const void* x, const void* y, void* out, int dtype, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out != nullptr, EISEN_E_ARG, "eisen_hip_mul: null out");
    EwArgs a{};
    a.in[0] = x;
    a.in[1] = y;
    a.out[0] = out;
    a.n = n;
    return dispatch_ew<OpMul>(ctx, dtype, a, "mul");
}

static int bcast_common(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, int rank,
                        const size_t* out_shape, const size_t* a_strides, const size_t* b_strides, bool mul) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, a && b && out && out_shape && a_strides && b_strides, EISEN_E_ARG, "bcast: null pointer");
    EISEN_REQUIRE(ctx, rank >= 1 && rank <= 4, EISEN_E_SHAPE, "bcast: rank %d not in 1..4", rank);
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "bcast: unknown dtype %d", dtype);
    BcastArgs g{};
    g.rank = rank;
    g.n = 1;
    for (int d = 0; d < rank; d++) {
        g.shape[d] = out_shape[d];
        g.sa[d] = a_strides[d];
        g.sb[d] = b_strides[d];
        g.n *= out_shape[d];
    }
    if (g.n == 0) return 0;
    const unsigned blocks = (unsigned)std::min<size_t>(4096, eisen_ceil_div(g.n, kEwThreads));
    if (dtype == EISEN_F32) {
        if (mul) bcast_kernel<float, true><<<blocks, kEwThreads, 0, ctx->stream>>>((const float*)a, (const float*)b, (float*)out, g);
        else bcast_kernel<float, false><<<blocks, kEwThreads, 0, ctx->stream>>>((const float*)a, (const float*)b, (float*)out, g);
    } else {
        if (mul) bcast_kernel<bf16_t, true><<<blocks, kEwThreads, 0, ctx->stream>>>((const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, g);
        else bcast_kernel<bf16_t, false><<<blocks, kEwThreads, 0, ctx->stream>>>((const bf16_t*)a, (const bf16_t*)b, (bf16_t*)out, g);
    }
    EISEN_LAUNCH_CHECK(ctx, "bcast_kernel");
    return 0;
}

extern "C" int eisen_hip_add_bcast(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, int rank,
                                   const size_t* out_shape, const size_t* a_strides, const size_t* b_strides) {
    return bcast_common(ctx, a, b, out, dtype, rank, out_shape, a_strides, b_strides, false);
}
extern "C" int eisen_hip_mul_bcast(eisen_ctx* ctx, const void* a, const void* b, void* out, int dtype, int rank,
                                   const size_t* out_shape, const size_t* a_strides, const size_t* b_strides) {
    return bcast_common(ctx, a, b, out, dtype, rank, out_shape, a_strides, b_strides, true);
}

static int bcast_backward_common(eisen_ctx* ctx, void* dst, const void* grad_out, const void* other, int dtype, bool dst_f32,
                                 int rank, const size_t* out_shape, const size_t* dst_strides,
                                 const size_t* other_strides, size_t dst_numel, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, dst && grad_out && out_shape && dst_strides, EISEN_E_ARG, "bcast_backward: null pointer");
    EISEN_REQUIRE(ctx, rank >= 1 && rank <= 4, EISEN_E_SHAPE, "bcast_backward: rank %d not in 1..4", rank);
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "bcast_backward: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, other == nullptr || other_strides != nullptr, EISEN_E_ARG, "bcast_backward: other without strides");
    BcastBwdArgs g{};
    g.rank = rank;
    g.dst_numel = dst_numel;
    size_t fixed = 1;
    for (int d = 0; d < rank; d++) {
        g.shape[d] = out_shape[d];
        g.sd[d] = dst_strides[d];
        g.so[d] = other ? other_strides[d] : 0;
        if (!(dst_strides[d] == 0 && out_shape[d] > 1)) fixed *= out_shape[d];
    }
    EISEN_REQUIRE(ctx, fixed == dst_numel, EISEN_E_SHAPE, "bcast_backward: dst_numel %zu does not match the non-broadcast dims (%zu)", dst_numel, fixed);
    if (dst_numel == 0) return 0;
    // one thread per dst element walks its whole reduction; when that leaves most of the chip idle (a handful of dst
    // elements, millions of terms each) the walk is cut into chunks of at least 1024 terms
    size_t total = 1;
    for (int d = 0; d < rank; d++) total *= out_shape[d];
    const size_t nred = total / dst_numel;
    size_t chunks = 1;
    if (dst_numel < 16384 && nred >= 8192) chunks = std::min<size_t>(nred / 1024, std::max<size_t>(1, 65536 / dst_numel));
    float* partial = nullptr;
    if (chunks > 1) {
        void* ws = nullptr;
        const int rc = eisen_workspace(ctx, dst_numel * chunks * sizeof(float), &ws);
        if (rc) return rc;
        partial = static_cast<float*>(ws);
    } else {
        chunks = 1;
    }
    const unsigned blocks = (unsigned)std::min<size_t>(4096, eisen_ceil_div(dst_numel * chunks, kEwThreads));
    const unsigned fin_blocks = (unsigned)std::min<size_t>(4096, eisen_ceil_div(dst_numel, kEwThreads));
    if (dtype == EISEN_F32) {
        bcast_bwd_kernel<float, float><<<blocks, kEwThreads, 0, ctx->stream>>>((float*)dst, (const float*)grad_out, (const float*)other, g, accumulate, chunks, partial);
        if (chunks > 1) bcast_bwd_finish_kernel<float><<<fin_blocks, kEwThreads, 0, ctx->stream>>>((float*)dst, partial, g, accumulate, chunks);
    } else if (dst_f32) {
        bcast_bwd_kernel<bf16_t, float><<<blocks, kEwThreads, 0, ctx->stream>>>((float*)dst, (const bf16_t*)grad_out, (const bf16_t*)other, g, accumulate, chunks, partial);
        if (chunks > 1) bcast_bwd_finish_kernel<float><<<fin_blocks, kEwThreads, 0, ctx->stream>>>((float*)dst, partial, g, accumulate, chunks);
    } else {
        bcast_bwd_kernel<bf16_t, bf16_t><<<blocks, kEwThreads, 0, ctx->stream>>>((bf16_t*)dst, (const bf16_t*)grad_out, (const bf16_t*)other, g, accumulate, chunks, partial);
        if (chunks > 1) bcast_bwd_finish_kernel<bf16_t><<<fin_blocks, kEwThreads, 0, ctx->stream>>>((bf16_t*)dst, partial, g, accumulate, chunks);
    }
    EISEN_LAUNCH_CHECK(ctx, "bcast_bwd_kernel");
    return 0;
}

extern "C" int eisen_hip_bcast_backward(eisen_ctx* ctx, void* dst, const void* grad_out, const void* other, int dtype,
                                        int rank, const size_t* out_shape, const size_t* dst_strides,
                                        const size_t* other_strides, size_t dst_numel, int accumulate) {
    return bcast_backward_common(ctx, dst, grad_out, other, dtype, false, rank, out_shape, dst_strides, other_strides, dst_numel, accumulate);
}

extern "C" int eisen_hip_bcast_backward_f32(eisen_ctx* ctx, float* dst, const void* grad_out, const void* other, int dtype,
                                            int rank, const size_t* out_shape, const size_t* dst_strides,
                                            const size_t* other_strides, size_t dst_numel, int accumulate) {
    return bcast_backward_common(ctx, dst, grad_out, other, dtype, true, rank, out_shape, dst_strides, other_strides, dst_numel, accumulate);
}

extern "C" int eisen_hip_mul_backward(eisen_ctx* ctx, const void* x, const void* y, const void* go, void* ga, void* gb,
                                      int dtype, size_t n, int accumulate_a, int accumulate_b) {
    EISEN_CHECK_CTX(ctx);
    EwArgs a{};
    a.in[0] = x;
    a.in[1] = y;
    a.in[2] = go;
    a.out[0] = ga;
    a.out[1] = gb;
    a.acc[0] = accumulate_a;
    a.acc[1] = accumulate_b;
    a.n = n;
    return dispatch_ew<OpMulBwd>(ctx, dtype, a, "mul_backward");
}

extern "C" int eisen_hip_silu(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out != nullptr, EISEN_E_ARG, "eisen_hip_silu: null out");
    EwArgs a{};
    a.in[0] = x;
    a.out[0] = out;
    a.n = n;
    return dispatch_ew<OpSilu>(ctx, dtype, a, "silu");
}

extern "C" int eisen_hip_silu_backward(eisen_ctx* ctx, const void* x, const void* go, void* gx, int dtype, size_t n,
                                       int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, gx != nullptr, EISEN_E_ARG, "eisen_hip_silu_backward: null gx");
    EwArgs a{};
    a.in[0] = x;
    a.in[1] = go;
    a.out[0] = gx;
    a.acc[0] = accumulate;
    a.n = n;
    return dispatch_ew<OpSiluBwd>(ctx, dtype, a, "silu_backward");
}

extern "C" int eisen_hip_swiglu(eisen_ctx* ctx, const void* gate, const void* up, void* out, int dtype, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out != nullptr, EISEN_E_ARG, "eisen_hip_swiglu: null out");
    EwArgs a{};
    a.in[0] = gate;
    a.in[1] = up;
    a.out[0] = out;
    a.n = n;
    return dispatch_ew<OpSwiglu>(ctx, dtype, a, "swiglu");
}

extern "C" int eisen_hip_swiglu_backward(eisen_ctx* ctx, const void* gate, const void* up, const void* go, void* dgate,
                                         void* dup, int dtype, size_t n, int accumulate_gate, int accumulate_up) {
    EISEN_CHECK_CTX(ctx);
    EwArgs a{};
    a.in[0] = gate;
    a.in[1] = up;
    a.in[2] = go;
    a.out[0] = dgate;
    a.out[1] = dup;
    a.acc[0] = accumulate_gate;
    a.acc[1] = accumulate_up;
    a.n = n;
    return dispatch_ew<OpSwigluBwd>(ctx, dtype, a, "swiglu_backward");
}
