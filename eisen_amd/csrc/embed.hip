// Embedding lookup and the deterministic embedding-gradient scatter.
#include <algorithm>
#include <numeric>

#include "device_utils.cuh"
#include "runtime.h"

namespace {

constexpr int kThreads = 256;

// out[i, :] = W[ids[i], :]   (src/graph/ops/transform.rs:296-303)
template <typename T, int N>
__global__ __launch_bounds__(kThreads) void gather_kernel(const T* __restrict__ w, const int32_t* __restrict__ ids,
                                                          T* __restrict__ out, size_t total_chunks, int chunks_per_row) {
    for (size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x; c < total_chunks; c += (size_t)gridDim.x * blockDim.x) {
        const size_t i = c / chunks_per_row;
        const int cc = (int)(c % chunks_per_row);
        const size_t row = (size_t)ids[i];
        if (N > 1)
            store_pack(out + c * N, load_pack(w + (row * chunks_per_row + cc) * N));
        else
            out[c] = w[row * chunks_per_row + cc];
    }
}

// One wave owns (one touched vocabulary row) x (one 64-packet column slab) and adds that
// row's occurrences in ascending position order, starting from the value already in gw:
//   gw[row] = ((gw[row] + go[i1]) + go[i2]) + ...      i1 < i2 < ...
// which is the CPU arm's order (src/graph/ops/transform.rs:309-314).  No atomics, so the
// result does not depend on scheduling.  Loads of the next occurrences are issued before the
// adds of the current ones (unroll 4) to keep several rows in flight.
template <typename T>
__global__ __launch_bounds__(kThreads) void scatter_rows_kernel(const T* __restrict__ go, float* __restrict__ gw,
                                                                const int32_t* __restrict__ seg_row,
                                                                const int32_t* __restrict__ seg_begin,
                                                                const int32_t* __restrict__ order, int n_segments,
                                                                int hidden, int slabs) {
    constexpr int N = Pack<T>::N;
    const int lane = threadIdx.x & 63;
    const size_t wave = (size_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x >> 6);
    const size_t seg = wave / slabs;
    if (seg >= (size_t)n_segments) return;
    const int col = ((int)(wave % slabs) * kWave + lane) * N;
    if (col >= hidden) return;
    const size_t row = (size_t)seg_row[seg];
    const int begin = seg_begin[seg], end = seg_begin[seg + 1];
    float acc[N];
    float* dst = gw + row * hidden + col;
#pragma unroll
    for (int j = 0; j < N; j += 4) {
        const float4 v = *reinterpret_cast<const float4*>(dst + j);
        acc[j] = v.x; acc[j + 1] = v.y; acc[j + 2] = v.z; acc[j + 3] = v.w;
    }
    int k = begin;
    for (; k + 4 <= end; k += 4) {
        Pack<T> p[4];
#pragma unroll
        for (int u = 0; u < 4; u++) p[u] = load_pack(go + (size_t)order[k + u] * hidden + col);
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int j = 0; j < N; j++) acc[j] += p[u].get(j);
    }
    for (; k < end; k++) {
        const Pack<T> p = load_pack(go + (size_t)order[k] * hidden + col);
#pragma unroll
        for (int j = 0; j < N; j++) acc[j] += p.get(j);
    }
#pragma unroll
    for (int j = 0; j < N; j += 4) *reinterpret_cast<float4*>(dst + j) = make_float4(acc[j], acc[j + 1], acc[j + 2], acc[j + 3]);
}

// Fallback for hidden sizes that are not packet multiples: one thread per (segment, column).
template <typename T>
__global__ __launch_bounds__(kThreads) void scatter_rows_scalar_kernel(const T* __restrict__ go, float* __restrict__ gw,
                                                                       const int32_t* __restrict__ seg_row,
                                                                       const int32_t* __restrict__ seg_begin,
                                                                       const int32_t* __restrict__ order, int n_segments,
                                                                       int hidden) {
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t seg = t / hidden;
    if (seg >= (size_t)n_segments) return;
    const int col = (int)(t % hidden);
    float acc = gw[(size_t)seg_row[seg] * hidden + col];
    for (int k = seg_begin[seg]; k < seg_begin[seg + 1]; k++) acc += to_f32(go[(size_t)order[k] * hidden + col]);
    gw[(size_t)seg_row[seg] * hidden + col] = acc;
}

}  // namespace

extern "C" int eisen_hip_gather(eisen_ctx* ctx, const void* weight, const int32_t* ids, void* out, int dtype,
                                size_t n_ids, size_t vocab, size_t hidden) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, weight && ids && out, EISEN_E_ARG, "gather: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "gather: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, vocab > 0 && vocab < (size_t(1) << 31) && hidden > 0 && hidden < (size_t(1) << 30), EISEN_E_SHAPE, "gather: vocab/hidden out of range");
    if (n_ids == 0) return 0;
    const size_t n = dtype == EISEN_F32 ? 4 : 8;
    const bool vec = hidden % n == 0 && eisen_aligned(weight, 16) && eisen_aligned(out, 16);
    const int cpr = (int)(vec ? hidden / n : hidden);
    const size_t chunks = n_ids * cpr;
    EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "gather_bf16" : "gather_f32", 2.0 * (double)n_ids * (double)hidden * eisen_dtype_size(dtype) + 4.0 * (double)n_ids);
    const unsigned blocks = (unsigned)std::min<size_t>(256 * 16, eisen_ceil_div(chunks, kThreads));
    if (dtype == EISEN_F32) {
        if (vec) gather_kernel<float, 4><<<blocks, kThreads, 0, ctx->stream>>>((const float*)weight, ids, (float*)out, chunks, cpr);
        else gather_kernel<float, 1><<<blocks, kThreads, 0, ctx->stream>>>((const float*)weight, ids, (float*)out, chunks, cpr);
    } else {
        if (vec) gather_kernel<bf16_t, 8><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)weight, ids, (bf16_t*)out, chunks, cpr);
        else gather_kernel<bf16_t, 1><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)weight, ids, (bf16_t*)out, chunks, cpr);
    }
    EISEN_LAUNCH_CHECK(ctx, "gather_kernel");
    return 0;
}

extern "C" int eisen_hip_gather_backward(eisen_ctx* ctx, const int32_t* ids_host, const void* go, float* gw, int dtype,
                                         size_t n_ids, size_t vocab, size_t hidden) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ids_host && go && gw, EISEN_E_ARG, "gather_backward: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "gather_backward: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, vocab > 0 && vocab < (size_t(1) << 31) && hidden > 0 && hidden < (size_t(1) << 30) && n_ids < (size_t(1) << 31),
                  EISEN_E_SHAPE, "gather_backward: sizes out of range");
    if (n_ids == 0) return 0;
    for (size_t i = 0; i < n_ids; i++)
        EISEN_REQUIRE(ctx, ids_host[i] >= 0 && (size_t)ids_host[i] < vocab, EISEN_E_ARG,
                      "gather_backward: id %d at position %zu outside [0, %zu)", ids_host[i], i, vocab);
    // stable order of positions by token id: ties keep ascending position
    std::vector<int32_t> order(n_ids);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return ids_host[a] < ids_host[b]; });
    std::vector<int32_t> seg_row, seg_begin;
    for (size_t k = 0; k < n_ids; k++)
        if (k == 0 || ids_host[order[k]] != ids_host[order[k - 1]]) {
            seg_row.push_back(ids_host[order[k]]);
            seg_begin.push_back((int32_t)k);
        }
    seg_begin.push_back((int32_t)n_ids);
    const size_t n_seg = seg_row.size();
    // one upload: [order | seg_row | seg_begin]
    const size_t total = n_ids + n_seg + (n_seg + 1);
    std::vector<int32_t> blob(total);
    std::copy(order.begin(), order.end(), blob.begin());
    std::copy(seg_row.begin(), seg_row.end(), blob.begin() + n_ids);
    std::copy(seg_begin.begin(), seg_begin.end(), blob.begin() + n_ids + n_seg);
    void* dev = nullptr;
    int rc = eisen_hip_malloc(ctx, total * sizeof(int32_t), &dev);
    if (rc) return rc;
    rc = eisen_hip_htod(ctx, dev, blob.data(), total * sizeof(int32_t));
    if (rc) {
        (void)eisen_hip_free(ctx, dev);
        return rc;
    }
    const int32_t* d_order = (const int32_t*)dev;
    const int32_t* d_row = d_order + n_ids;
    const int32_t* d_begin = d_row + n_seg;
    const size_t n = dtype == EISEN_F32 ? 4 : 8;
    const bool vec = hidden % n == 0 && eisen_aligned(go, 16) && eisen_aligned(gw, 16);
    // algorithmic bytes: every row of dOut read once, every touched row of the f32 gradient read and written once
    EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "scatter_rows_bf16" : "scatter_rows_f32",
                        (double)n_ids * (double)hidden * eisen_dtype_size(dtype) + 8.0 * (double)n_seg * (double)hidden + 4.0 * (double)total);
    if (vec) {
        const int slabs = (int)eisen_ceil_div(hidden, (size_t)kWave * n);
        const size_t waves = n_seg * slabs;
        const unsigned blocks = (unsigned)eisen_ceil_div(waves, kThreads / kWave);
        if (dtype == EISEN_F32)
            scatter_rows_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)go, gw, d_row, d_begin, d_order, (int)n_seg, (int)hidden, slabs);
        else
            scatter_rows_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)go, gw, d_row, d_begin, d_order, (int)n_seg, (int)hidden, slabs);
        EISEN_LAUNCH_CHECK(ctx, "scatter_rows_kernel");
    } else {
        const unsigned blocks = (unsigned)eisen_ceil_div(n_seg * hidden, kThreads);
        if (dtype == EISEN_F32)
            scatter_rows_scalar_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)go, gw, d_row, d_begin, d_order, (int)n_seg, (int)hidden);
        else
            scatter_rows_scalar_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)go, gw, d_row, d_begin, d_order, (int)n_seg, (int)hidden);
        EISEN_LAUNCH_CHECK(ctx, "scatter_rows_scalar_kernel");
    }
    return eisen_hip_free(ctx, dev);  // stream-ordered: the block is reused only by later work
}
