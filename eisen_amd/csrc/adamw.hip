// Fused multi-tensor AdamW over f32 master weights, global gradient norm, zero_grad.
// One launch covers every parameter tensor: a device table of slots plus a prefix table of
// 16-byte-packet chunks maps each workgroup to its tensor.  HBM-bound: 16 B read each of
// w, g, m, v and 16 B written each of w, m, v per packet (+ 8 B for the bf16 copy).
#include "device_utils.cuh"
#include "runtime.h"

namespace {

constexpr int kThreads = 256;
constexpr int kChunk = kThreads * 4 * 4;  // elements per workgroup: 4 float4 packets per thread

struct SlotDev {
    float* w;
    const float* g;
    float* m;
    float* v;
    bf16_t* wb;
    unsigned long long n;
    unsigned long long first_block;  // index of this tensor's first workgroup
};

__device__ __forceinline__ int find_slot(const SlotDev* __restrict__ slots, int n_slots, unsigned block) {
    int lo = 0, hi = n_slots - 1;  // last slot with first_block <= block
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (slots[mid].first_block <= block) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));
// streaming access: optimizer state is touched once per step and never reused from cache
__device__ __forceinline__ float4 nt_load4(const float* p) {
    const f32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
    return make_float4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ void nt_store4(float* p, float4 v) {
    f32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<f32x4_t*>(p));
}

struct AdamParams {
    float lr, beta1, beta2, eps, wd, bc1, bc2;
};

// src/nn/optim.rs:533-542: decayed = w(1 - lr*wd); m = b1 m + (1-b1) g; v = b2 v + (1-b2) g g;
// w = decayed - lr*(m*bc1)/(sqrt(v*bc2) + eps)
__device__ __forceinline__ void adam_elem(float& w, float g, float& m, float& v, const AdamParams& p) {
    const float decayed = w * (1.0f - p.lr * p.wd);
    m = p.beta1 * m + (1.0f - p.beta1) * g;
    v = p.beta2 * v + (1.0f - p.beta2) * g * g;
    const float m_hat = m * p.bc1;
    const float v_hat = v * p.bc2;
    w = decayed - p.lr * m_hat / (sqrtf(v_hat) + p.eps);
}

__global__ __launch_bounds__(kThreads) void adamw_kernel(const SlotDev* __restrict__ slots, int n_slots, AdamParams p,
                                                         const float* __restrict__ grad_scale) {
    const int si = find_slot(slots, n_slots, blockIdx.x);
    const SlotDev s = slots[si];
    const size_t base = (size_t)(blockIdx.x - s.first_block) * kChunk;
    const float gs = grad_scale ? grad_scale[0] : 1.0f;
    const bool vec = (s.n % 4 == 0);  // tensors come from the 256-byte-granule pool: bases are aligned
    if (vec) {
        // all 16 loads of the thread are issued before the first use: 16 KB per stream and workgroup in flight
        float4 w[4], g[4], m[4], v[4];
        bool on[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
            on[u] = e < s.n;
            if (on[u]) {
                w[u] = nt_load4(s.w + e);
                g[u] = nt_load4(s.g + e);
                m[u] = nt_load4(s.m + e);
                v[u] = nt_load4(s.v + e);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (!on[u]) continue;
            const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
            adam_elem(w[u].x, g[u].x * gs, m[u].x, v[u].x, p);
            adam_elem(w[u].y, g[u].y * gs, m[u].y, v[u].y, p);
            adam_elem(w[u].z, g[u].z * gs, m[u].z, v[u].z, p);
            adam_elem(w[u].w, g[u].w * gs, m[u].w, v[u].w, p);
            nt_store4(s.w + e, w[u]);
            nt_store4(s.m + e, m[u]);
            nt_store4(s.v + e, v[u]);
            if (s.wb) {
                bf16x4 b;
                b[0] = (bf16_t)w[u].x; b[1] = (bf16_t)w[u].y; b[2] = (bf16_t)w[u].z; b[3] = (bf16_t)w[u].w;
                *reinterpret_cast<bf16x4*>(s.wb + e) = b;
            }
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
        if (e >= s.n) break;
        for (int j = 0; j < 4 && e + j < s.n; j++) {
            float w = s.w[e + j], m = s.m[e + j], v = s.v[e + j];
            adam_elem(w, s.g[e + j] * gs, m, v, p);
            s.w[e + j] = w; s.m[e + j] = m; s.v[e + j] = v;
            if (s.wb) s.wb[e + j] = (bf16_t)w;
        }
    }
}

__global__ __launch_bounds__(kThreads) void zero_grads_kernel(const SlotDev* __restrict__ slots, int n_slots) {
    const int si = find_slot(slots, n_slots, blockIdx.x);
    const SlotDev s = slots[si];
    const size_t base = (size_t)(blockIdx.x - s.first_block) * kChunk;
    float* g = const_cast<float*>(s.g);
    const bool vec = (s.n % 4 == 0);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
        if (e >= s.n) break;
        if (vec) *reinterpret_cast<float4*>(g + e) = make_float4(0.f, 0.f, 0.f, 0.f);
        else
            for (int j = 0; j < 4 && e + j < s.n; j++) g[e + j] = 0.f;
    }
}

// stage 1: one f64 partial per workgroup (src/nn/optim.rs:258-262 accumulates x*x in f64)
__global__ __launch_bounds__(kThreads) void sumsq_kernel(const SlotDev* __restrict__ slots, int n_slots, double* __restrict__ partial) {
    __shared__ double sh[kThreads / kWave];
    const int si = find_slot(slots, n_slots, blockIdx.x);
    const SlotDev s = slots[si];
    const size_t base = (size_t)(blockIdx.x - s.first_block) * kChunk;
    double acc = 0.0;
    if (s.n % 4 == 0) {
        float4 g[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
            g[u] = e < s.n ? *reinterpret_cast<const float4*>(s.g + e) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            acc += (double)g[u].x * (double)g[u].x;
            acc += (double)g[u].y * (double)g[u].y;
            acc += (double)g[u].z * (double)g[u].z;
            acc += (double)g[u].w * (double)g[u].w;
        }
    } else {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const size_t e = base + ((size_t)u * kThreads + threadIdx.x) * 4;
            if (e >= s.n) break;
            for (int j = 0; j < 4 && e + j < s.n; j++) {
                const double x = (double)s.g[e + j];
                acc += x * x;
            }
        }
    }
    acc = wave_sum_f64(acc);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int k = 0; k < kThreads / kWave; k++) t += sh[k];
        partial[blockIdx.x] = t;
    }
}
// stage 2: one workgroup, fixed order; writes norm and clip coefficient (src/nn/optim.rs:282-287)
__global__ __launch_bounds__(1024) void norm_finish_kernel(const double* __restrict__ partial, size_t n, float max_norm, float* __restrict__ out) {
    __shared__ double sh[1024 / kWave];
    double acc = 0.0;
    for (size_t i = threadIdx.x; i < n; i += 1024) acc += partial[i];
    acc = wave_sum_f64(acc);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int k = 0; k < 1024 / kWave; k++) t += sh[k];
        const float norm = (float)sqrt(t);
        float coef = 1.0f;
        if (norm > 0.0f) coef = fminf(max_norm / (norm + 1e-6f), 1.0f);
        out[0] = norm;
        out[1] = coef;
    }
}

// Uploads the slot table; returns the device copy and the total workgroup count.
int upload_slots(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots, bool need_moments, SlotDev** dev_out,
                 size_t* blocks_out, const char* who) {
    EISEN_REQUIRE(ctx, slots && n_slots > 0 && n_slots < (size_t(1) << 20), EISEN_E_ARG, "%s: bad slot table", who);
    std::vector<SlotDev> host(n_slots);
    size_t blocks = 0;
    for (size_t i = 0; i < n_slots; i++) {
        const eisen_param_slot& s = slots[i];
        EISEN_REQUIRE(ctx, s.g && s.n > 0, EISEN_E_ARG, "%s: slot %zu has a null gradient or zero size", who, i);
        EISEN_REQUIRE(ctx, !need_moments || (s.w && s.m && s.v), EISEN_E_ARG, "%s: slot %zu lacks w/m/v", who, i);
        EISEN_REQUIRE(ctx, eisen_aligned(s.g, 16) && eisen_aligned(s.w, 16) && eisen_aligned(s.m, 16) && eisen_aligned(s.v, 16) && eisen_aligned(s.w_bf16, 8),
                      EISEN_E_ALIGN, "%s: slot %zu buffers must be 16-byte aligned", who, i);
        host[i] = SlotDev{s.w, s.g, s.m, s.v, (bf16_t*)s.w_bf16, (unsigned long long)s.n, (unsigned long long)blocks};
        blocks += eisen_ceil_div(s.n, kChunk);
    }
    EISEN_REQUIRE(ctx, blocks < (size_t(1) << 31), EISEN_E_SHAPE, "%s: too many elements for one launch", who);
    void* dev = nullptr;
    int rc = eisen_hip_malloc(ctx, n_slots * sizeof(SlotDev), &dev);
    if (rc) return rc;
    rc = eisen_hip_htod(ctx, dev, host.data(), n_slots * sizeof(SlotDev));
    if (rc) {
        (void)eisen_hip_free(ctx, dev);
        return rc;
    }
    *dev_out = (SlotDev*)dev;
    *blocks_out = blocks;
    return 0;
}

}  // namespace

extern "C" int eisen_hip_adamw_step(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots, float lr, float beta1,
                                    float beta2, float eps, float weight_decay, float bc1, float bc2,
                                    const float* grad_scale_device) {
    EISEN_CHECK_CTX(ctx);
    SlotDev* dev = nullptr;
    size_t blocks = 0;
    int rc = upload_slots(ctx, slots, n_slots, true, &dev, &blocks, "adamw_step");
    if (rc) return rc;
    AdamParams p{lr, beta1, beta2, eps, weight_decay, bc1, bc2};
    double bytes = 0.0;  // per parameter: w, g, m, v read, w, m, v written (28 B) and the bf16 copy written where there is one
    for (size_t i = 0; i < n_slots; i++) bytes += (double)slots[i].n * (slots[i].w_bf16 ? 30.0 : 28.0);
    EisenProfScope prof(ctx, "adamw", bytes);
    adamw_kernel<<<(unsigned)blocks, kThreads, 0, ctx->stream>>>(dev, (int)n_slots, p, grad_scale_device);
    EISEN_LAUNCH_CHECK(ctx, "adamw_kernel");
    return eisen_hip_free(ctx, dev);
}

extern "C" int eisen_hip_zero_grads(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots) {
    EISEN_CHECK_CTX(ctx);
    SlotDev* dev = nullptr;
    size_t blocks = 0;
    int rc = upload_slots(ctx, slots, n_slots, false, &dev, &blocks, "zero_grads");
    if (rc) return rc;
    zero_grads_kernel<<<(unsigned)blocks, kThreads, 0, ctx->stream>>>(dev, (int)n_slots);
    EISEN_LAUNCH_CHECK(ctx, "zero_grads_kernel");
    return eisen_hip_free(ctx, dev);
}

extern "C" int eisen_hip_grad_norm(eisen_ctx* ctx, const eisen_param_slot* slots, size_t n_slots, float max_norm,
                                   float* out_device) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, out_device != nullptr, EISEN_E_ARG, "grad_norm: null output");
    SlotDev* dev = nullptr;
    size_t blocks = 0;
    int rc = upload_slots(ctx, slots, n_slots, false, &dev, &blocks, "grad_norm");
    if (rc) return rc;
    void* ws = nullptr;
    rc = eisen_workspace(ctx, blocks * sizeof(double), &ws);
    if (rc) {
        (void)eisen_hip_free(ctx, dev);
        return rc;
    }
    double bytes = 0.0;
    for (size_t i = 0; i < n_slots; i++) bytes += (double)slots[i].n * 4.0;
    EisenProfScope prof(ctx, "grad_sumsq", bytes);
    sumsq_kernel<<<(unsigned)blocks, kThreads, 0, ctx->stream>>>(dev, (int)n_slots, (double*)ws);
    EISEN_LAUNCH_CHECK(ctx, "sumsq_kernel");
    norm_finish_kernel<<<1, 1024, 0, ctx->stream>>>((const double*)ws, blocks, max_norm, out_device);
    EISEN_LAUNCH_CHECK(ctx, "norm_finish_kernel");
    return eisen_hip_free(ctx, dev);
}
