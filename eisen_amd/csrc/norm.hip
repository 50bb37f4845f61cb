// RMSNorm forward/backward and row softmax forward/backward.
// One 64-lane wave owns one row; lanes stride the row in 16-byte packets so every global
// access is a fully coalesced 1 KiB wave transaction.  Reductions are wave shuffles.
#include "device_utils.cuh"
#include "runtime.h"

namespace {

constexpr int kRowThreads = 256;  // 4 waves = 4 rows per block
constexpr int kRowWaves = kRowThreads / kWave;
constexpr int kBwdThreads = 512;  // backward: 8 waves per block share one partial-dw row
constexpr int kBwdWaves = kBwdThreads / kWave;

// y = x * rrms * w,  rrms = 1/sqrt(mean(x^2) + eps)   (src/graph/ops/normalization.rs:141-151)
template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void rms_norm_fwd_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                                                   T* __restrict__ out, float* __restrict__ rrms_out,
                                                                   size_t rows, int dim, float eps) {
    constexpr int N = VEC ? Pack<T>::N : 1;
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * kRowWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * dim;
    T* orow = out + row * dim;
    float ss = 0.f;
    for (int c = lane * N; c < dim; c += kWave * N) {
        if (VEC) {
            const Pack<T> p = load_pack(xr + c);
#pragma unroll
            for (int j = 0; j < N; j++) ss += p.get(j) * p.get(j);
        } else {
            const float v = to_f32(xr[c]);
            ss += v * v;
        }
    }
    ss = wave_sum(ss);
    const float rrms = 1.0f / sqrtf(ss / (float)dim + eps);
    if (lane == 0) rrms_out[row] = rrms;
    for (int c = lane * N; c < dim; c += kWave * N) {
        if (VEC) {
            const Pack<T> p = load_pack(xr + c);  // second read of a row this wave just streamed: L2/TCP hit
            Pack<T> o;
#pragma unroll
            for (int j = 0; j < N; j += 4) {
                const float4 g4 = *reinterpret_cast<const float4*>(w + c + j);
                o.set(j, p.get(j) * rrms * g4.x);
                o.set(j + 1, p.get(j + 1) * rrms * g4.y);
                o.set(j + 2, p.get(j + 2) * rrms * g4.z);
                o.set(j + 3, p.get(j + 3) * rrms * g4.w);
            }
            store_pack(orow + c, o);
        } else {
            orow[c] = from_f32<T>(to_f32(xr[c]) * rrms * w[c]);
        }
    }
}

// dx = rrms*(go*w) - x*(rrms^3/D)*sum_d(go*x*w);  dw_partial[d] += go*x*rrms
// (src/graph/ops/normalization.rs:157-171).  Each wave walks rows wave_id, wave_id+W, ...
// and keeps its dw partial in registers; partials meet in LDS and leave as one row of
// `partial` per block.  A second kernel sums the block rows in fixed order.
template <typename T, int MAXP>
__global__ __launch_bounds__(kBwdThreads) void rms_norm_bwd_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                                                   const float* __restrict__ rrms_in,
                                                                   const T* __restrict__ go, const T* gx_old, T* gx,
                                                                   float* __restrict__ partial, size_t rows, int dim) {
    // gx_old: what dx is added to (gx itself for an in-place accumulation, another buffer of the same layout, or null to assign)
    const bool accumulate_x = gx_old != nullptr;
    constexpr int N = Pack<T>::N;
    extern __shared__ float lds[];  // [kBwdWaves][dim]
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const size_t wave_global = (size_t)blockIdx.x * kBwdWaves + wid;
    const size_t wave_stride = (size_t)gridDim.x * kBwdWaves;
    float dw[MAXP][N];
#pragma unroll
    for (int p = 0; p < MAXP; p++)
#pragma unroll
        for (int j = 0; j < N; j++) dw[p][j] = 0.f;

    // a lane owns the same columns in every row: its gains live in registers
    float wv[MAXP][N];
#pragma unroll
    for (int p = 0; p < MAXP; p++) {
        const int c = (p * kWave + lane) * N;
#pragma unroll
        for (int j = 0; j < N; j += 4) {
            const float4 t = c < dim ? *reinterpret_cast<const float4*>(w + c + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            wv[p][j] = t.x; wv[p][j + 1] = t.y; wv[p][j + 2] = t.z; wv[p][j + 3] = t.w;
        }
    }
    // the next row's packets are requested before the current row is reduced, so a wave always has
    // two rows of loads in flight
    // (the row of gx an accumulating call adds to travels with them: requested after the row reduction it would cost
    // every row a second memory latency)
    Pack<T> xp[MAXP], gp[MAXP], op[MAXP], xn[MAXP], gn[MAXP], on[MAXP];
    auto fetch = [&](size_t row, Pack<T>* xd, Pack<T>* gd, Pack<T>* od) {
#pragma unroll
        for (int p = 0; p < MAXP; p++) {
            const int c = (p * kWave + lane) * N;
            if (c < dim) {
                xd[p] = load_pack(x + row * dim + c);
                gd[p] = load_pack(go + row * dim + c);
                if (accumulate_x) od[p] = load_pack(gx_old + row * dim + c);
            }
        }
    };
    if (wave_global < rows) fetch(wave_global, xp, gp, op);
    for (size_t row = wave_global; row < rows; row += wave_stride) {
        T* gxr = gx + row * dim;
        const float rrms = rrms_in[row];
        const size_t next = row + wave_stride;
        if (next < rows) fetch(next, xn, gn, on);
        float gdxw = 0.f;
#pragma unroll
        for (int p = 0; p < MAXP; p++) {
            const int c = (p * kWave + lane) * N;
            if (c < dim) {
#pragma unroll
                for (int j = 0; j < N; j++) gdxw += gp[p].get(j) * xp[p].get(j) * wv[p][j];
            }
        }
        gdxw = wave_sum(gdxw);
        const float rrc_d = rrms * rrms * rrms / (float)dim;
#pragma unroll
        for (int p = 0; p < MAXP; p++) {
            const int c = (p * kWave + lane) * N;
            if (c < dim) {
                Pack<T> o = op[p];
#pragma unroll
                for (int j = 0; j < N; j++) {
                    const float xv = xp[p].get(j), gv = gp[p].get(j);
                    const float dx = rrms * (gv * wv[p][j]) - xv * rrc_d * gdxw;
                    o.set(j, accumulate_x ? o.get(j) + dx : dx);
                    dw[p][j] += gv * xv * rrms;
                }
                store_pack(gxr + c, o);
            }
        }
#pragma unroll
        for (int p = 0; p < MAXP; p++) {
            xp[p] = xn[p];
            gp[p] = gn[p];
            op[p] = on[p];
        }
    }
    // combine the block's waves in a fixed order
#pragma unroll
    for (int p = 0; p < MAXP; p++) {
        const int c = (p * kWave + lane) * N;
        if (c < dim)
#pragma unroll
            for (int j = 0; j < N; j++) lds[wid * dim + c + j] = dw[p][j];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < dim; c += kBwdThreads) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < kBwdWaves; k++) s += lds[k * dim + c];
        partial[(size_t)blockIdx.x * dim + c] = s;
    }
}

// Second stage: gw[c] += sum over the block rows of `partial`, in a fixed order.  A workgroup owns
// 32 columns; its 8 row groups each add every 8th partial row, then meet in LDS (group 0..7 in order).
// blockIdx.y picks one of up to kFinishSlots (partial, gw) pairs: the gains of many norms finish in one launch.
constexpr int kFinishSlots = 64;
struct FinishSlots {
    const float* partial[kFinishSlots];
    float* gw[kFinishSlots];
    int nrows[kFinishSlots];
    int assign[kFinishSlots];  // 1: gw = sum (a gradient whose clearing is still pending), 0: gw += sum
};
__global__ __launch_bounds__(256) void rms_norm_dw_reduce_kernel(FinishSlots slots, int dim) {
    __shared__ float sh[8][32];
    const float* __restrict__ partial = slots.partial[blockIdx.y];
    float* __restrict__ gw = slots.gw[blockIdx.y];
    const int nblocks = slots.nrows[blockIdx.y];
    const int cl = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int c = blockIdx.x * 32 + cl;
    float s = 0.f;
    if (c < dim)
#pragma unroll 8
        for (int b = rg; b < nblocks; b += 8) s += partial[(size_t)b * dim + c];
    sh[rg][cl] = s;
    __syncthreads();
    if (rg == 0 && c < dim) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) t += sh[k][cl];
        gw[c] = (slots.assign[blockIdx.y] ? 0.f : gw[c]) + t;
    }
}

// Scalar fallback for rows that are not packet-aligned: one wave per row, same arithmetic.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void rms_norm_bwd_scalar_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                                                          const float* __restrict__ rrms_in,
                                                                          const T* __restrict__ go, const T* gx_old, T* gx,
                                                                          size_t rows, int dim) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * kRowWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * dim;
    const T* gr = go + row * dim;
    T* gxr = gx + row * dim;
    const float rrms = rrms_in[row];
    float gdxw = 0.f;
    for (int c = lane; c < dim; c += kWave) gdxw += to_f32(gr[c]) * to_f32(xr[c]) * w[c];
    gdxw = wave_sum(gdxw);
    const float rrc_d = rrms * rrms * rrms / (float)dim;
    for (int c = lane; c < dim; c += kWave) {
        const float dx = rrms * (to_f32(gr[c]) * w[c]) - to_f32(xr[c]) * rrc_d * gdxw;
        gxr[c] = from_f32<T>(gx_old ? to_f32(gx_old[row * dim + c]) + dx : dx);
    }
}
// dw for the scalar fallback: one thread per column walks the rows in order.
template <typename T>
__global__ void rms_norm_dw_scalar_kernel(const T* __restrict__ x, const float* __restrict__ rrms_in,
                                          const T* __restrict__ go, float* __restrict__ gw, size_t rows, int dim) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= dim) return;
    float s = 0.f;
    for (size_t r = 0; r < rows; r++) s += to_f32(go[r * dim + c]) * to_f32(x[r * dim + c]) * rrms_in[r];
    gw[c] += s;
}

// softmax over the last dim (src/graph/ops/reduction.rs:483-496): max, exp(x-max), divide.
template <typename T>
__global__ __launch_bounds__(kRowThreads) void softmax_fwd_kernel(const T* __restrict__ x, T* __restrict__ out, size_t rows,
                                                                  int n) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * kRowWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * n;
    T* orow = out + row * n;
    float mx = -INFINITY;
    for (int c = lane; c < n; c += kWave) mx = fmaxf(mx, to_f32(xr[c]));
    mx = wave_max(mx);
    float sum = 0.f;
    for (int c = lane; c < n; c += kWave) sum += __expf(to_f32(xr[c]) - mx);
    sum = wave_sum(sum);
    for (int c = lane; c < n; c += kWave) orow[c] = from_f32<T>(__expf(to_f32(xr[c]) - mx) / sum);
}

// gx += y*(go - sum(go*y))   (src/graph/ops/reduction.rs:504-512)
template <typename T>
__global__ __launch_bounds__(kRowThreads) void softmax_bwd_kernel(const T* __restrict__ y, const T* __restrict__ go,
                                                                  T* __restrict__ gx, size_t rows, int n, int accumulate) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * kRowWaves + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* yr = y + row * n;
    const T* gr = go + row * n;
    T* gxr = gx + row * n;
    float dot = 0.f;
    for (int c = lane; c < n; c += kWave) dot += to_f32(gr[c]) * to_f32(yr[c]);
    dot = wave_sum(dot);
    for (int c = lane; c < n; c += kWave) {
        const float v = to_f32(yr[c]) * (to_f32(gr[c]) - dot);
        gxr[c] = from_f32<T>(accumulate ? to_f32(gxr[c]) + v : v);
    }
}

template <typename T>
int rms_norm_fwd(eisen_ctx* ctx, const void* x, const float* w, void* out, float* rrms, size_t rows, size_t dim, float eps) {
    const unsigned blocks = (unsigned)eisen_ceil_div(rows, kRowWaves);
    const bool vec = dim % Pack<T>::N == 0 && eisen_aligned(x, 16) && eisen_aligned(out, 16) && eisen_aligned(w, 16);
    // algorithmic bytes: x read, y written, one rrms per row
    EisenProfScope prof(ctx, sizeof(T) == 2 ? "rms_norm_fwd_bf16" : "rms_norm_fwd_f32", 2.0 * (double)rows * (double)dim * sizeof(T) + 4.0 * (double)rows);
    if (vec)
        rms_norm_fwd_kernel<T, true><<<blocks, kRowThreads, 0, ctx->stream>>>((const T*)x, w, (T*)out, rrms, rows, (int)dim, eps);
    else
        rms_norm_fwd_kernel<T, false><<<blocks, kRowThreads, 0, ctx->stream>>>((const T*)x, w, (T*)out, rrms, rows, (int)dim, eps);
    EISEN_LAUNCH_CHECK(ctx, "rms_norm_fwd_kernel");
    return 0;
}

constexpr unsigned kMaxPartialRows = EISEN_RMS_NORM_PARTIAL_ROWS;

template <typename T, int MAXP>
int rms_norm_bwd_vec(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, const void* gx_old, void* gx, float* partial,
                     unsigned blocks, size_t rows, size_t dim) {
    const size_t lds = (size_t)kBwdWaves * dim * sizeof(float);
    rms_norm_bwd_kernel<T, MAXP><<<blocks, kBwdThreads, lds, ctx->stream>>>((const T*)x, w, rrms, (const T*)go, (const T*)gx_old, (T*)gx, partial, rows,
                                                                            (int)dim);
    EISEN_LAUNCH_CHECK(ctx, "rms_norm_bwd_kernel");
    return 0;
}

// dx, and the gain gradient as rows of `partial` ([kMaxPartialRows][dim]); *nrows = rows written.
template <typename T>
int rms_norm_bwd_partial(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, const void* gx_old, void* gx, float* partial,
                         size_t* nrows, size_t rows, size_t dim) {
    constexpr int N = Pack<T>::N;
    const bool accumulate_x = gx_old != nullptr;
    const bool vec = dim % N == 0 && eisen_aligned(x, 16) && eisen_aligned(go, 16) && eisen_aligned(gx, 16) && eisen_aligned(gx_old, 16) && eisen_aligned(w, 16) &&
                     dim <= (size_t)kWave * N * 8 && (size_t)kBwdWaves * dim * sizeof(float) <= 64 * 1024;
    // algorithmic bytes: x and dy read, dx written (and read first when the call accumulates), one rrms per row
    EisenProfScope prof(ctx, sizeof(T) == 2 ? "rms_norm_bwd_bf16" : "rms_norm_bwd_f32",
                        (accumulate_x ? 4.0 : 3.0) * (double)rows * (double)dim * sizeof(T) + 4.0 * (double)rows);
    if (vec) {
        // enough waves to cover the chip a few times over, few enough that the partial rows stay small
        const unsigned blocks = (unsigned)std::min<size_t>(eisen_ceil_div(rows, kBwdWaves), kMaxPartialRows);
        *nrows = blocks;
        const size_t packs = eisen_ceil_div(dim, (size_t)kWave * N);
        if (packs <= 1) return rms_norm_bwd_vec<T, 1>(ctx, x, w, rrms, go, gx_old, gx, partial, blocks, rows, dim);
        if (packs <= 2) return rms_norm_bwd_vec<T, 2>(ctx, x, w, rrms, go, gx_old, gx, partial, blocks, rows, dim);
        if (packs <= 4) return rms_norm_bwd_vec<T, 4>(ctx, x, w, rrms, go, gx_old, gx, partial, blocks, rows, dim);
        return rms_norm_bwd_vec<T, 8>(ctx, x, w, rrms, go, gx_old, gx, partial, blocks, rows, dim);
    }
    rms_norm_bwd_scalar_kernel<T><<<(unsigned)eisen_ceil_div(rows, kRowWaves), kRowThreads, 0, ctx->stream>>>(
        (const T*)x, w, rrms, (const T*)go, (const T*)gx_old, (T*)gx, rows, (int)dim);
    EISEN_LAUNCH_CHECK(ctx, "rms_norm_bwd_scalar_kernel");
    *nrows = 1;  // one thread per column adds its rows in order into a zeroed row
    int rc = eisen_hip_fill(ctx, partial, EISEN_F32, 0.0f, dim);
    if (rc) return rc;
    rms_norm_dw_scalar_kernel<T><<<(unsigned)eisen_ceil_div(dim, 256), 256, 0, ctx->stream>>>((const T*)x, rrms, (const T*)go, partial, rows, (int)dim);
    EISEN_LAUNCH_CHECK(ctx, "rms_norm_dw_scalar_kernel");
    return 0;
}

int rms_norm_dw_finish(eisen_ctx* ctx, size_t n, const float* const* partial, float* const* gw, const size_t* nrows, size_t dim, const int* assign) {
    double bytes = 0.0;
    for (size_t i = 0; i < n; i++) bytes += ((double)nrows[i] + 2.0) * (double)dim * 4.0;
    EisenProfScope prof(ctx, "rms_norm_dw_finish", bytes);
    for (size_t first = 0; first < n; first += kFinishSlots) {
        FinishSlots slots{};
        const size_t m = std::min<size_t>(kFinishSlots, n - first);
        for (size_t i = 0; i < m; i++) {
            slots.partial[i] = partial[first + i];
            slots.gw[i] = gw[first + i];
            slots.nrows[i] = (int)nrows[first + i];
            slots.assign[i] = assign ? assign[first + i] : 0;
        }
        rms_norm_dw_reduce_kernel<<<dim3((unsigned)eisen_ceil_div(dim, 32), (unsigned)m, 1), 256, 0, ctx->stream>>>(slots, (int)dim);
        EISEN_LAUNCH_CHECK(ctx, "rms_norm_dw_reduce_kernel");
    }
    return 0;
}

}  // namespace

extern "C" int eisen_hip_rms_norm(eisen_ctx* ctx, const void* x, const float* w, void* out, float* rrms, int dtype,
                                  size_t rows, size_t dim, float eps) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, x && w && out && rrms, EISEN_E_ARG, "eisen_hip_rms_norm: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_rms_norm: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, dim > 0 && dim < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_rms_norm: dim %zu out of range", dim);
    if (rows == 0) return 0;
    return dtype == EISEN_F32 ? rms_norm_fwd<float>(ctx, x, w, out, rrms, rows, dim, eps)
                              : rms_norm_fwd<bf16_t>(ctx, x, w, out, rrms, rows, dim, eps);
}

extern "C" int eisen_hip_rms_norm_backward(eisen_ctx* ctx, const void* x, const float* w, const float* rrms,
                                           const void* go, void* gx, float* gw, int dtype, size_t rows, size_t dim,
                                           int accumulate_x) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, x && w && rrms && go && gx && gw, EISEN_E_ARG, "eisen_hip_rms_norm_backward: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_rms_norm_backward: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, dim > 0 && dim < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_rms_norm_backward: dim %zu out of range", dim);
    if (rows == 0) return 0;
    // the two-part form with the library's workspace in between
    void* ws = nullptr;
    int rc = eisen_workspace(ctx, (size_t)kMaxPartialRows * dim * sizeof(float), &ws);
    if (rc) return rc;
    size_t nrows = 0;
    const void* gx_old = accumulate_x ? gx : nullptr;
    rc = dtype == EISEN_F32 ? rms_norm_bwd_partial<float>(ctx, x, w, rrms, go, gx_old, gx, (float*)ws, &nrows, rows, dim)
                            : rms_norm_bwd_partial<bf16_t>(ctx, x, w, rrms, go, gx_old, gx, (float*)ws, &nrows, rows, dim);
    if (rc) return rc;
    const float* p = (const float*)ws;
    return rms_norm_dw_finish(ctx, 1, &p, &gw, &nrows, dim, nullptr);
}

extern "C" int eisen_hip_rms_norm_backward_partial(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, void* gx,
                                                   float* partial, size_t* nrows_out, int dtype, size_t rows, size_t dim, int accumulate_x) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, x && w && rrms && go && gx && partial && nrows_out, EISEN_E_ARG, "eisen_hip_rms_norm_backward_partial: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_rms_norm_backward_partial: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, dim > 0 && dim < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_rms_norm_backward_partial: dim %zu out of range", dim);
    *nrows_out = 0;
    if (rows == 0) return 0;
    const void* gx_old = accumulate_x ? gx : nullptr;
    return dtype == EISEN_F32 ? rms_norm_bwd_partial<float>(ctx, x, w, rrms, go, gx_old, gx, partial, nrows_out, rows, dim)
                              : rms_norm_bwd_partial<bf16_t>(ctx, x, w, rrms, go, gx_old, gx, partial, nrows_out, rows, dim);
}

extern "C" int eisen_hip_rms_norm_backward_partial_add(eisen_ctx* ctx, const void* x, const float* w, const float* rrms, const void* go, const void* gx_in,
                                                       void* gx, float* partial, size_t* nrows_out, int dtype, size_t rows, size_t dim) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, x && w && rrms && go && gx_in && gx && partial && nrows_out, EISEN_E_ARG, "eisen_hip_rms_norm_backward_partial_add: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_rms_norm_backward_partial_add: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, dim > 0 && dim < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_rms_norm_backward_partial_add: dim %zu out of range", dim);
    *nrows_out = 0;
    if (rows == 0) return 0;
    return dtype == EISEN_F32 ? rms_norm_bwd_partial<float>(ctx, x, w, rrms, go, gx_in, gx, partial, nrows_out, rows, dim)
                              : rms_norm_bwd_partial<bf16_t>(ctx, x, w, rrms, go, gx_in, gx, partial, nrows_out, rows, dim);
}

extern "C" int eisen_hip_rms_norm_dw_finish(eisen_ctx* ctx, size_t n, const float* const* partial, float* const* gw, const size_t* nrows, size_t dim,
                                            const int* assign) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, n == 0 || (partial && gw && nrows), EISEN_E_ARG, "eisen_hip_rms_norm_dw_finish: null pointer");
    EISEN_REQUIRE(ctx, dim > 0 && dim < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_rms_norm_dw_finish: dim %zu out of range", dim);
    for (size_t i = 0; i < n; i++) {
        EISEN_REQUIRE(ctx, partial[i] && gw[i] && nrows[i] <= kMaxPartialRows, EISEN_E_ARG, "eisen_hip_rms_norm_dw_finish: entry %zu is null or has too many rows", i);
        for (size_t j = 0; j < i; j++) EISEN_REQUIRE(ctx, gw[i] != gw[j], EISEN_E_ARG, "eisen_hip_rms_norm_dw_finish: entries %zu and %zu add to the same gradient", j, i);
    }
    return rms_norm_dw_finish(ctx, n, partial, gw, nrows, dim, assign);
}

extern "C" int eisen_hip_softmax(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t rows, size_t n) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, x && out, EISEN_E_ARG, "eisen_hip_softmax: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_softmax: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, n > 0 && n < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_softmax: n %zu out of range", n);
    if (rows == 0) return 0;
    const unsigned blocks = (unsigned)eisen_ceil_div(rows, kRowWaves);
    if (dtype == EISEN_F32)
        softmax_fwd_kernel<float><<<blocks, kRowThreads, 0, ctx->stream>>>((const float*)x, (float*)out, rows, (int)n);
    else
        softmax_fwd_kernel<bf16_t><<<blocks, kRowThreads, 0, ctx->stream>>>((const bf16_t*)x, (bf16_t*)out, rows, (int)n);
    EISEN_LAUNCH_CHECK(ctx, "softmax_fwd_kernel");
    return 0;
}

extern "C" int eisen_hip_softmax_backward(eisen_ctx* ctx, const void* out, const void* go, void* gx, int dtype,
                                          size_t rows, size_t n, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out && go && gx, EISEN_E_ARG, "eisen_hip_softmax_backward: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_softmax_backward: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, n > 0 && n < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_softmax_backward: n %zu out of range", n);
    if (rows == 0) return 0;
    const unsigned blocks = (unsigned)eisen_ceil_div(rows, kRowWaves);
    if (dtype == EISEN_F32)
        softmax_bwd_kernel<float><<<blocks, kRowThreads, 0, ctx->stream>>>((const float*)out, (const float*)go, (float*)gx, rows, (int)n, accumulate);
    else
        softmax_bwd_kernel<bf16_t><<<blocks, kRowThreads, 0, ctx->stream>>>((const bf16_t*)out, (const bf16_t*)go, (bf16_t*)gx, rows, (int)n, accumulate);
    EISEN_LAUNCH_CHECK(ctx, "softmax_bwd_kernel");
    return 0;
}
