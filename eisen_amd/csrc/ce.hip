// Fused softmax-cross-entropy forward+backward: one read of the logits, one write of dLogits.
//
// One workgroup owns one row.  The row is loaded once with 16-byte packets and stays in
// registers (VPT packets per lane, widened to f32) across the three phases: row max (+ first
// argmax when asked for), exponentials (computed once, kept) and their sum, gradient write.  Reductions are wave64 shuffles plus one LDS exchange
// between the block's waves.  The row is read and its gradient written with streaming (non-temporal) accesses: each byte
// is touched once, and keeping it out of the caches' way is worth 4-5 % at 8192 x 32000.  Per-row losses go to a buffer; a second one-block kernel sums
// them in a fixed order, so the loss carries no float atomics and is reproducible.
//
// Follows Graph::cross_entropy / cross_entropy_masked (src/graph/ops/reduction.rs:676-706,
// :897-931): p = exp(x - max) / sum, loss_row = -ln(p_t + 1e-8), dlogit = (p - onehot) * scale.
#include "device_utils.cuh"
#include "runtime.h"

namespace {

struct ArgMax {
    float v;
    int i;
};
__device__ __forceinline__ ArgMax argmax_combine(ArgMax a, ArgMax b) {
    // first index of the maximum wins on ties
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}
__device__ __forceinline__ ArgMax wave_argmax(ArgMax a) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        ArgMax b;
        b.v = __shfl_xor(a.v, o, 64);
        b.i = __shfl_xor(a.i, o, 64);
        a = argmax_combine(a, b);
    }
    return a;
}

template <typename T, int THREADS, int VPT, bool WANT_ARGMAX>
__global__ __launch_bounds__(THREADS) void ce_fused_kernel(const T* __restrict__ logits, const int32_t* __restrict__ targets,
                                                           T* __restrict__ dlogits, float* __restrict__ row_loss,
                                                           int32_t* __restrict__ argmax_out, float* __restrict__ target_logit_out,
                                                           int classes, float scale) {
    constexpr int N = Pack<T>::N;
    constexpr int W = THREADS / kWave;
    constexpr float kLog2e = 1.4426950408889634f;
    __shared__ float s_f[W];
    __shared__ int s_i[W];
    const size_t row = blockIdx.x;
    const int target = targets[row];
    const T* xr = logits + row * classes;
    T* gr = dlogits + row * classes;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;

    // masked row: zero gradient, no loss (src/graph/ops/reduction.rs:898, :925).  A target beyond the
    // class count (the reference would panic on the index) is treated the same way: the host
    // validates targets before upload, the device only has to stay inside the row.
    if (target < 0 || target >= classes) {
        Pack<T> z;
#pragma unroll
        for (int j = 0; j < N; j++) z.set(j, 0.f);
#pragma unroll
        for (int v = 0; v < VPT; v++) {
            const int c = (v * THREADS + threadIdx.x) * N;
            if (c < classes) store_pack(gr + c, z);
        }
        if (threadIdx.x == 0) {
            row_loss[row] = 0.f;
            if (argmax_out) argmax_out[row] = -1;
            if (target_logit_out) target_logit_out[row] = 0.f;
        }
        return;
    }

    // phase 1: the row comes in once (VPT packets per lane, all loads in flight together) and stays in
    // registers in its storage type: half the registers of an f32 copy, so twice the workgroups per CU
    // keep loads in flight.  Running maximum (and, when asked for, its first index).
    Pack<T> raw[VPT];
    ArgMax am{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        const int c = (v * THREADS + threadIdx.x) * N;
        if (c < classes) raw[v] = load_pack_streaming(xr + c);
    }
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        const int c = (v * THREADS + threadIdx.x) * N;
        if (c < classes) {
#pragma unroll
            for (int j = 0; j < N; j++) {
                const float xv = raw[v].get(j);
                if (WANT_ARGMAX) {
                    if (xv > am.v) {  // ascending c within the lane: strict > keeps the first
                        am.v = xv;
                        am.i = c + j;
                    }
                } else {
                    am.v = fmaxf(am.v, xv);
                }
            }
        }
    }
    if (WANT_ARGMAX) {
        am = wave_argmax(am);
        if (W > 1) {
            if (lane == 0) {
                s_f[wid] = am.v;
                s_i[wid] = am.i;
            }
            __syncthreads();
            am = ArgMax{s_f[0], s_i[0]};
#pragma unroll
            for (int k = 1; k < W; k++) am = argmax_combine(am, ArgMax{s_f[k], s_i[k]});
            __syncthreads();
        }
    } else {
        am.v = block_max<THREADS>(am.v, s_f);
    }
    const float mx = am.v;

    // phase 2: row sum of e = 2^(x*log2e - max*log2e).  The exponent is never positive, so the bare
    // hardware exp2 (results below 2^-126 flush to zero) is exact enough.
    const float bias = -mx * kLog2e;
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        const int c = (v * THREADS + threadIdx.x) * N;
        if (c < classes) {
#pragma unroll
            for (int j = 0; j < N; j++) sum += __builtin_amdgcn_exp2f(fmaf(raw[v].get(j), kLog2e, bias));
        }
    }
    sum = block_sum<THREADS>(sum, s_f);
    const float inv = 1.0f / sum;
    const float gscale = inv * scale;

    // phase 3: dlogit = (e/sum - onehot) * scale with e recomputed (a second exp2 costs less than the
    // registers that keeping it would take); the lane that holds the target fixes its element up and
    // writes the row loss
#pragma unroll
    for (int v = 0; v < VPT; v++) {
        const int c = (v * THREADS + threadIdx.x) * N;
        if (c < classes) {
            Pack<T> g;
            const bool has_target = target >= c && target < c + N;
#pragma unroll
            for (int j = 0; j < N; j++) {
                const float xv = raw[v].get(j);
                const float e = __builtin_amdgcn_exp2f(fmaf(xv, kLog2e, bias));
                float gv = e * gscale;
                if (has_target && c + j == target) {
                    row_loss[row] = -logf(e * inv + 1e-8f);
                    if (target_logit_out) target_logit_out[row] = xv;
                    gv -= scale;
                }
                g.set(j, gv);
            }
            store_pack_streaming(gr + c, g);
        }
    }
    if (WANT_ARGMAX && threadIdx.x == 0 && argmax_out) argmax_out[row] = am.i;
}

// Generic row kernel for class counts that do not fit the register-resident variants or
// are not packet multiples: three passes over the row (the 2nd and 3rd hit L2).
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void ce_generic_kernel(const T* __restrict__ logits, const int32_t* __restrict__ targets,
                                                             T* __restrict__ dlogits, float* __restrict__ row_loss,
                                                             int32_t* __restrict__ argmax_out, float* __restrict__ target_logit_out,
                                                             int classes, float scale) {
    constexpr int W = THREADS / kWave;
    __shared__ float s_f[W];
    __shared__ int s_i[W];
    const size_t row = blockIdx.x;
    const int target = targets[row];
    const T* xr = logits + row * classes;
    T* gr = dlogits + row * classes;
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    if (target < 0 || target >= classes) {
        for (int c = threadIdx.x; c < classes; c += THREADS) gr[c] = from_f32<T>(0.f);
        if (threadIdx.x == 0) {
            row_loss[row] = 0.f;
            if (argmax_out) argmax_out[row] = -1;
            if (target_logit_out) target_logit_out[row] = 0.f;
        }
        return;
    }
    ArgMax am{-INFINITY, 0x7fffffff};
    for (int c = threadIdx.x; c < classes; c += THREADS) {
        const float f = to_f32(xr[c]);
        if (f > am.v) {
            am.v = f;
            am.i = c;
        }
    }
    am = wave_argmax(am);
    if (W > 1) {
        if (lane == 0) {
            s_f[wid] = am.v;
            s_i[wid] = am.i;
        }
        __syncthreads();
        am = ArgMax{s_f[0], s_i[0]};
        for (int k = 1; k < W; k++) am = argmax_combine(am, ArgMax{s_f[k], s_i[k]});
        __syncthreads();
    }
    const float mx = am.v;
    float sum = 0.f;
    for (int c = threadIdx.x; c < classes; c += THREADS) sum += __expf(to_f32(xr[c]) - mx);
    sum = block_sum<THREADS>(sum, s_f);
    const float inv = 1.0f / sum;
    for (int c = threadIdx.x; c < classes; c += THREADS) {
        const float xv = to_f32(xr[c]);
        float p = __expf(xv - mx) * inv;
        if (c == target) {
            row_loss[row] = -logf(p + 1e-8f);
            if (target_logit_out) target_logit_out[row] = xv;
            p -= 1.0f;
        }
        gr[c] = from_f32<T>(p * scale);
    }
    if (threadIdx.x == 0 && argmax_out) argmax_out[row] = am.i;
}

// loss = normalizer * sum_rows row_loss, summed by one block in a fixed order.
__global__ __launch_bounds__(1024) void ce_loss_reduce_kernel(const float* __restrict__ row_loss, float* __restrict__ loss_out,
                                                              size_t rows, float normalizer) {
    __shared__ float s[1024 / kWave];
    float acc = 0.f;
    for (size_t r = threadIdx.x; r < rows; r += 1024) acc += row_loss[r];
    acc = block_sum<1024>(acc, s);
    if (threadIdx.x == 0) loss_out[0] = acc * normalizer;
}

template <typename T, int THREADS, int VPT>
void launch_fused(eisen_ctx* ctx, const void* logits, const int32_t* targets, void* dlogits, float* row_loss,
                  int32_t* argmax_out, float* target_logit_out, size_t rows, size_t classes, float scale) {
    if (argmax_out)
        ce_fused_kernel<T, THREADS, VPT, true><<<dim3((unsigned)rows), dim3(THREADS), 0, ctx->stream>>>(
            (const T*)logits, targets, (T*)dlogits, row_loss, argmax_out, target_logit_out, (int)classes, scale);
    else
        ce_fused_kernel<T, THREADS, VPT, false><<<dim3((unsigned)rows), dim3(THREADS), 0, ctx->stream>>>(
            (const T*)logits, targets, (T*)dlogits, row_loss, argmax_out, target_logit_out, (int)classes, scale);
}

template <typename T>
int ce_dispatch(eisen_ctx* ctx, const void* logits, const int32_t* targets, void* dlogits, float* row_loss,
                int32_t* argmax_out, float* target_logit_out, size_t rows, size_t classes, float scale) {
    constexpr int N = Pack<T>::N;
    const bool vec = classes % N == 0 && eisen_aligned(logits, 16) && eisen_aligned(dlogits, 16);
    const size_t packets = classes / N;
#define CE_ARGS ctx, logits, targets, dlogits, row_loss, argmax_out, target_logit_out, rows, classes, scale
    if (vec && packets <= 256 * 1) launch_fused<T, 256, 1>(CE_ARGS);
    else if (vec && packets <= 256 * 2) launch_fused<T, 256, 2>(CE_ARGS);
    else if (vec && packets <= 256 * 4) launch_fused<T, 256, 4>(CE_ARGS);
    else if (vec && packets <= 512 * 4) launch_fused<T, 512, 4>(CE_ARGS);
    else if (vec && packets <= 512 * 8) launch_fused<T, 512, 8>(CE_ARGS);
    else if (vec && packets <= 1024 * 8) launch_fused<T, 1024, 8>(CE_ARGS);
    else
        ce_generic_kernel<T, 512><<<dim3((unsigned)rows), dim3(512), 0, ctx->stream>>>(
            (const T*)logits, targets, (T*)dlogits, row_loss, argmax_out, target_logit_out, (int)classes, scale);
#undef CE_ARGS
    EISEN_LAUNCH_CHECK(ctx, "ce kernel");
    return 0;
}

}  // namespace

extern "C" int eisen_hip_cross_entropy(eisen_ctx* ctx, const void* logits, const int32_t* targets, void* dlogits,
                                       float* row_loss, float* loss_out, int32_t* argmax_out, float* target_logit_out,
                                       int dtype, size_t rows, size_t classes, float normalizer, float grad_scale) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, logits && targets && dlogits && row_loss && loss_out, EISEN_E_ARG, "cross_entropy: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "cross_entropy: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, rows > 0 && rows < (size_t(1) << 31), EISEN_E_SHAPE, "cross_entropy: rows %zu out of range", rows);
    EISEN_REQUIRE(ctx, classes > 0 && classes < (size_t(1) << 30), EISEN_E_SHAPE, "cross_entropy: classes %zu out of range", classes);
    const float scale = normalizer * grad_scale;
    // algorithmic bytes: logits read once, dlogits written once, targets read, row losses written
    EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "ce_fused_bf16" : "ce_fused_f32",
                        2.0 * (double)rows * (double)classes * (double)eisen_dtype_size(dtype) + 8.0 * (double)rows);
    int rc = dtype == EISEN_F32
                 ? ce_dispatch<float>(ctx, logits, targets, dlogits, row_loss, argmax_out, target_logit_out, rows, classes, scale)
                 : ce_dispatch<bf16_t>(ctx, logits, targets, dlogits, row_loss, argmax_out, target_logit_out, rows, classes, scale);
    if (rc) return rc;
    ce_loss_reduce_kernel<<<1, 1024, 0, ctx->stream>>>(row_loss, loss_out, rows, normalizer);
    EISEN_LAUNCH_CHECK(ctx, "ce_loss_reduce_kernel");
    return 0;
}
