// Rotary embedding forward/backward (interleaved pairs) and the [b,s,h,d] <-> [b,h,s,d]
// permutation / GQA head repeat.  HBM-bound; 16-byte packets per lane.
#include <cmath>

#include "device_utils.cuh"
#include "runtime.h"

// cos/sin table [seq][head_dim/2] as float2, built on the host with the libm routines the CPU
// arm uses (theta = pos / 10000^(2p/hd); src/graph/ops/transform.rs:559-561), so the device
// rotates by exactly the same angles.
int eisen_rope_table_get(eisen_ctx* ctx, size_t seq, size_t head_dim, const float2** out) {
    for (auto& t : ctx->rope_tables)
        if (t.head_dim == head_dim && t.seq >= seq) {
            *out = reinterpret_cast<const float2*>(t.cos_sin);
            return 0;
        }
    const size_t half = head_dim / 2;
    const size_t bytes = seq * half * sizeof(float2);
    std::vector<float2> host(seq * half);
    for (size_t pos = 0; pos < seq; pos++)
        for (size_t p = 0; p < half; p++) {
            const float theta = (float)pos / powf(10000.0f, (2.0f * (float)p) / (float)head_dim);
            host[pos * half + p] = make_float2(cosf(theta), sinf(theta));
        }
    float* dev = nullptr;
    ctx->driver_allocs++;
    EISEN_HIP_TRY(ctx, hipMallocAsync((void**)&dev, bytes, ctx->stream));
    EISEN_HIP_TRY(ctx, hipMemcpyAsync(dev, host.data(), bytes, hipMemcpyHostToDevice, ctx->stream));
    EISEN_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // `host` dies at return
    eisen_rope_table t;
    t.seq = seq;
    t.head_dim = head_dim;
    t.cos_sin = dev;
    ctx->rope_tables.push_back(t);
    *out = reinterpret_cast<const float2*>(dev);
    return 0;
}

namespace {

constexpr int kThreads = 256;

// fwd: y0 = x0 c - x1 s, y1 = x0 s + x1 c;  bwd: dx0 = g0 c + g1 s, dx1 = -g0 s + g1 c
// (src/graph/ops/transform.rs:562-566, :592-595).  One packet = N/2 pairs of one head.
template <typename T, bool BWD>
__global__ __launch_bounds__(kThreads) void rope_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                        const float2* __restrict__ table, size_t n_packets, int seq,
                                                        int hidden, int head_dim, int accumulate) {
    constexpr int N = Pack<T>::N;
    const int half = head_dim / 2;
    const int packets_per_row = hidden / N;
    for (size_t pk = (size_t)blockIdx.x * blockDim.x + threadIdx.x; pk < n_packets; pk += (size_t)gridDim.x * blockDim.x) {
        const size_t row = pk / packets_per_row;           // b*seq + pos
        const int col = (int)(pk % packets_per_row) * N;    // first element of the packet
        const int pos = (int)(row % seq);
        const int pair0 = (col % head_dim) / 2;
        const Pack<T> v = load_pack(in + pk * N);
        Pack<T> o;
        if (accumulate) o = load_pack(out + pk * N);
#pragma unroll
        for (int j = 0; j < N / 2; j++) {
            const float2 cs = table[(size_t)pos * half + pair0 + j];
            const float a = v.get(2 * j), b = v.get(2 * j + 1);
            float r0, r1;
            if (BWD) {
                r0 = a * cs.x + b * cs.y;
                r1 = -a * cs.y + b * cs.x;
            } else {
                rope_rotate_forward(a, b, cs, r0, r1);
            }
            o.set(2 * j, accumulate ? o.get(2 * j) + r0 : r0);
            o.set(2 * j + 1, accumulate ? o.get(2 * j + 1) + r1 : r1);
        }
        store_pack(out + pk * N, o);
    }
}

// The forward rotation of two tensors that share batch, seq and head_dim (the q and k projections of an attention block)
// as one launch: packets [0, n0) belong to the first tensor, the rest to the second.
template <typename T>
__global__ __launch_bounds__(kThreads) void rope_pair_kernel(const T* __restrict__ in0, T* __restrict__ out0, size_t n0, int hidden0,
                                                             const T* __restrict__ in1, T* __restrict__ out1, size_t n1, int hidden1,
                                                             const float2* __restrict__ table, int seq, int head_dim) {
    constexpr int N = Pack<T>::N;
    const int half = head_dim / 2;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n0 + n1; i += (size_t)gridDim.x * blockDim.x) {
        const bool second = i >= n0;
        const size_t pk = second ? i - n0 : i;
        const T* in = second ? in1 : in0;
        T* out = second ? out1 : out0;
        const int packets_per_row = (second ? hidden1 : hidden0) / N;
        const size_t row = pk / packets_per_row;
        const int col = (int)(pk % packets_per_row) * N;
        const int pos = (int)(row % seq);
        const int pair0 = (col % head_dim) / 2;
        const Pack<T> v = load_pack(in + pk * N);
        Pack<T> o;
#pragma unroll
        for (int j = 0; j < N / 2; j++) {
            const float2 cs = table[(size_t)pos * half + pair0 + j];
            const float a = v.get(2 * j), b = v.get(2 * j + 1);
            float r0, r1;
            rope_rotate_forward(a, b, cs, r0, r1);
            o.set(2 * j, r0);
            o.set(2 * j + 1, r1);
        }
        store_pack(out + pk * N, o);
    }
}

template <typename T, bool BWD>
int launch_rope(eisen_ctx* ctx, const void* in, void* out, size_t batch, size_t seq, size_t hidden, size_t head_dim,
                int accumulate) {
    constexpr int N = Pack<T>::N;
    const float2* table = nullptr;
    int rc = eisen_rope_table_get(ctx, seq, head_dim, &table);
    if (rc) return rc;
    const size_t n_packets = batch * seq * hidden / N;
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(n_packets, kThreads));
    rope_kernel<T, BWD><<<blocks, kThreads, 0, ctx->stream>>>((const T*)in, (T*)out, table, n_packets, (int)seq, (int)hidden,
                                                              (int)head_dim, accumulate);
    EISEN_LAUNCH_CHECK(ctx, "rope_kernel");
    return 0;
}

int rope_common(eisen_ctx* ctx, const void* in, void* out, int dtype, size_t batch, size_t seq, size_t hidden,
                size_t head_dim, int accumulate, bool bwd) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, in && out, EISEN_E_ARG, "rope: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "rope: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, head_dim >= 2 && head_dim % 2 == 0 && hidden % head_dim == 0, EISEN_E_SHAPE,
                  "rope: hidden %zu must be a multiple of an even head_dim (%zu)", hidden, head_dim);
    const size_t n = dtype == EISEN_F32 ? 4 : 8;
    EISEN_REQUIRE(ctx, head_dim % n == 0, EISEN_E_SHAPE, "rope: head_dim %zu must be a multiple of %zu for this dtype", head_dim, n);
    EISEN_REQUIRE(ctx, eisen_aligned(in, 16) && eisen_aligned(out, 16), EISEN_E_ALIGN, "rope: buffers must be 16-byte aligned");
    EISEN_REQUIRE(ctx, seq < (size_t(1) << 24) && hidden < (size_t(1) << 24), EISEN_E_SHAPE, "rope: seq/hidden too large");
    if (batch * seq * hidden == 0) return 0;
    if (dtype == EISEN_F32)
        return bwd ? launch_rope<float, true>(ctx, in, out, batch, seq, hidden, head_dim, accumulate)
                   : launch_rope<float, false>(ctx, in, out, batch, seq, hidden, head_dim, accumulate);
    return bwd ? launch_rope<bf16_t, true>(ctx, in, out, batch, seq, hidden, head_dim, accumulate)
               : launch_rope<bf16_t, false>(ctx, in, out, batch, seq, hidden, head_dim, accumulate);
}

// out[b,h,s,:] (+)= in[b,s,h,:]   (src/graph/ops/transform.rs:87-114); the backward is the same
// kernel with (s,h) swapped.  D-contiguous chunks move as packets when aligned.
template <typename T, int N>
__global__ __launch_bounds__(kThreads) void transpose_0213_kernel(const T* __restrict__ in, T* __restrict__ out, size_t total_chunks,
                                                                  int s, int h, int chunks_per_d, int accumulate) {
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < total_chunks; c += (size_t)gridDim.x * blockDim.x) {
        // c indexes the input in [b, s, h, d/N] order
        const int dc = (int)(c % chunks_per_d);
        size_t r = c / chunks_per_d;
        const int hh = (int)(r % h);
        r /= h;
        const int ss = (int)(r % s);
        const size_t bb = r / s;
        const size_t oc = ((bb * h + hh) * s + ss) * chunks_per_d + dc;
        if (N > 1) {
            const Pack<T> v = load_pack(in + c * N);
            Pack<T> o = v;
            if (accumulate) {
                o = load_pack(out + oc * N);
#pragma unroll
                for (int j = 0; j < Pack<T>::N; j++) o.set(j, o.get(j) + v.get(j));
            }
            store_pack(out + oc * N, o);
        } else {
            out[oc] = from_f32<T>(accumulate ? to_f32(out[oc]) + to_f32(in[c]) : to_f32(in[c]));
        }
    }
}

// out[b, kv*rep + r, s, :] = in[b, kv, s, :]   (src/graph/ops/gqa.rs:147-160)
template <typename T>
__global__ __launch_bounds__(kThreads) void repeat_kv_kernel(const T* __restrict__ in, T* __restrict__ out, size_t total_out,
                                                             size_t head_elems, int kv_heads, int repeats) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_out; i += (size_t)gridDim.x * blockDim.x) {
        const size_t e = i % head_elems;
        const size_t qh_flat = i / head_elems;  // b*qh + q
        const size_t q = qh_flat % ((size_t)kv_heads * repeats);
        const size_t b = qh_flat / ((size_t)kv_heads * repeats);
        out[i] = in[(b * kv_heads + q / repeats) * head_elems + e];
    }
}
// gin[b,kv,s,:] (+)= sum_{r ascending} go[b, kv*rep + r, s, :]   (src/graph/ops/gqa.rs:168-184)
template <typename T>
__global__ __launch_bounds__(kThreads) void repeat_kv_bwd_kernel(const T* __restrict__ go, T* __restrict__ gin, size_t total_in,
                                                                 size_t head_elems, int kv_heads, int repeats, int accumulate) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_in; i += (size_t)gridDim.x * blockDim.x) {
        const size_t e = i % head_elems;
        const size_t kv_flat = i / head_elems;  // b*kv + kv
        const size_t kv = kv_flat % kv_heads;
        const size_t b = kv_flat / kv_heads;
        float acc = accumulate ? to_f32(gin[i]) : 0.f;
        for (int r = 0; r < repeats; r++)
            acc += to_f32(go[((b * kv_heads + kv) * repeats + r) * head_elems + e]);
        gin[i] = from_f32<T>(acc);
    }
}

}  // namespace

extern "C" int eisen_hip_rope(eisen_ctx* ctx, const void* x, void* out, int dtype, size_t batch, size_t seq, size_t hidden,
                              size_t head_dim) {
    return rope_common(ctx, x, out, dtype, batch, seq, hidden, head_dim, 0, false);
}
extern "C" int eisen_hip_rope_pair(eisen_ctx* ctx, const void* q, void* q_out, size_t hidden_q, const void* k, void* k_out, size_t hidden_k, int dtype,
                                   size_t batch, size_t seq, size_t head_dim) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, q && q_out && k && k_out, EISEN_E_ARG, "rope_pair: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "rope_pair: unknown dtype %d", dtype);
    const size_t n = dtype == EISEN_F32 ? 4 : 8;
    const bool one_launch = head_dim >= 2 && head_dim % n == 0 && hidden_q % head_dim == 0 && hidden_k % head_dim == 0 && hidden_q > 0 && hidden_k > 0 &&
                            batch * seq > 0 && seq < (size_t(1) << 24) && hidden_q < (size_t(1) << 24) && hidden_k < (size_t(1) << 24) &&
                            eisen_aligned(q, 16) && eisen_aligned(q_out, 16) && eisen_aligned(k, 16) && eisen_aligned(k_out, 16);
    if (!one_launch) {  // the single-tensor entry point validates and reports
        const int rc = eisen_hip_rope(ctx, q, q_out, dtype, batch, seq, hidden_q, head_dim);
        return rc ? rc : eisen_hip_rope(ctx, k, k_out, dtype, batch, seq, hidden_k, head_dim);
    }
    const float2* table = nullptr;
    const int rc = eisen_rope_table_get(ctx, seq, head_dim, &table);
    if (rc) return rc;
    const size_t n0 = batch * seq * hidden_q / n, n1 = batch * seq * hidden_k / n;
    // algorithmic bytes: every element read once and written once
    EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "rope_pair_bf16" : "rope_pair_f32", 2.0 * (double)(n0 + n1) * 16.0);
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(n0 + n1, kThreads));
    if (dtype == EISEN_F32)
        rope_pair_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)q, (float*)q_out, n0, (int)hidden_q, (const float*)k, (float*)k_out, n1,
                                                                      (int)hidden_k, table, (int)seq, (int)head_dim);
    else
        rope_pair_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)q, (bf16_t*)q_out, n0, (int)hidden_q, (const bf16_t*)k, (bf16_t*)k_out,
                                                                       n1, (int)hidden_k, table, (int)seq, (int)head_dim);
    EISEN_LAUNCH_CHECK(ctx, "rope_pair_kernel");
    return 0;
}

extern "C" int eisen_hip_rope_backward(eisen_ctx* ctx, const void* go, void* gx, int dtype, size_t batch, size_t seq,
                                       size_t hidden, size_t head_dim, int accumulate) {
    return rope_common(ctx, go, gx, dtype, batch, seq, hidden, head_dim, accumulate, true);
}

extern "C" int eisen_hip_transpose_0213(eisen_ctx* ctx, const void* in, void* out, int dtype, size_t b, size_t s, size_t h,
                                        size_t d, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, in && out, EISEN_E_ARG, "transpose_0213: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "transpose_0213: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, s < (size_t(1) << 30) && h < (size_t(1) << 30) && d < (size_t(1) << 30), EISEN_E_SHAPE, "transpose_0213: dims too large");
    const size_t total = b * s * h * d;
    if (total == 0) return 0;
    const size_t n = dtype == EISEN_F32 ? 4 : 8;
    const bool vec = d % n == 0 && eisen_aligned(in, 16) && eisen_aligned(out, 16);
    const size_t chunks = vec ? total / n : total;
    const int cpd = (int)(vec ? d / n : d);
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(chunks, kThreads));
    if (dtype == EISEN_F32) {
        if (vec) transpose_0213_kernel<float, 4><<<blocks, kThreads, 0, ctx->stream>>>((const float*)in, (float*)out, chunks, (int)s, (int)h, cpd, accumulate);
        else transpose_0213_kernel<float, 1><<<blocks, kThreads, 0, ctx->stream>>>((const float*)in, (float*)out, chunks, (int)s, (int)h, cpd, accumulate);
    } else {
        if (vec) transpose_0213_kernel<bf16_t, 8><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)in, (bf16_t*)out, chunks, (int)s, (int)h, cpd, accumulate);
        else transpose_0213_kernel<bf16_t, 1><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)in, (bf16_t*)out, chunks, (int)s, (int)h, cpd, accumulate);
    }
    EISEN_LAUNCH_CHECK(ctx, "transpose_0213_kernel");
    return 0;
}

extern "C" int eisen_hip_repeat_kv(eisen_ctx* ctx, const void* in, void* out, int dtype, size_t batch, size_t kv_heads,
                                   size_t seq, size_t head_dim, size_t repeats) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, in && out, EISEN_E_ARG, "repeat_kv: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "repeat_kv: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, repeats >= 1 && kv_heads * repeats < (size_t(1) << 20), EISEN_E_SHAPE, "repeat_kv: bad head counts");
    const size_t total = batch * kv_heads * repeats * seq * head_dim;
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(total, kThreads));
    if (dtype == EISEN_F32)
        repeat_kv_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)in, (float*)out, total, seq * head_dim, (int)kv_heads, (int)repeats);
    else
        repeat_kv_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)in, (bf16_t*)out, total, seq * head_dim, (int)kv_heads, (int)repeats);
    EISEN_LAUNCH_CHECK(ctx, "repeat_kv_kernel");
    return 0;
}

extern "C" int eisen_hip_repeat_kv_backward(eisen_ctx* ctx, const void* go, void* gin, int dtype, size_t batch,
                                            size_t kv_heads, size_t seq, size_t head_dim, size_t repeats, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, go && gin, EISEN_E_ARG, "repeat_kv_backward: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "repeat_kv_backward: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, repeats >= 1 && kv_heads * repeats < (size_t(1) << 20), EISEN_E_SHAPE, "repeat_kv_backward: bad head counts");
    const size_t total = batch * kv_heads * seq * head_dim;
    if (total == 0) return 0;
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(total, kThreads));
    if (dtype == EISEN_F32)
        repeat_kv_bwd_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)go, (float*)gin, total, seq * head_dim, (int)kv_heads, (int)repeats, accumulate);
    else
        repeat_kv_bwd_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)go, (bf16_t*)gin, total, seq * head_dim, (int)kv_heads, (int)repeats, accumulate);
    EISEN_LAUNCH_CHECK(ctx, "repeat_kv_bwd_kernel");
    return 0;
}
