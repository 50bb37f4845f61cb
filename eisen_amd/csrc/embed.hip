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

// ---- position index built on the device ---------------------------------------------------------
// Keys id * n_pow2 + position are unique, so sorting them is the stable sort of the positions by id.  One workgroup of
// 1024 threads sorts 1024 * R of them (R = 1..16) with a bitonic network whose keys stay in registers: thread t holds
// elements t, t + 1024, ...; a compare-exchange at distance j >= 1024 pairs two registers of one thread, j < 64 two
// lanes of one wave (a shuffle), and only the distances 64..512 go through LDS (18 to 26 of the 55 to 105 steps).  The
// kernel writes the ids and positions in key order; ids outside [0, vocab) get the padding key and drop out.
constexpr int kSortThreads = 1024, kSortMax = 16384;
template <int R>
__global__ __launch_bounds__(kSortThreads) void scatter_sort_kernel(const int32_t* __restrict__ ids, int n, int shift, int vocab,
                                                                   int32_t* __restrict__ sorted_ids, int32_t* __restrict__ order,
                                                                   int32_t* __restrict__ run_end) {
    constexpr int NP = kSortThreads * R;
    __shared__ unsigned keys[NP];
    const int tid = threadIdx.x;
    unsigned key[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int i = r * kSortThreads + tid;
        unsigned v = 0xffffffffu;
        if (i < n) {
            const int id = ids[i];
            if (id >= 0 && id < vocab) v = ((unsigned)id << shift) | (unsigned)i;
        }
        key[r] = v;
    }
#pragma unroll
    for (int k = 2; k <= NP; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            if (j >= kSortThreads) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int rp = r ^ (j / kSortThreads);
                    if (rp > r) {  // registers r and rp of this thread: element r * 1024 + tid is the lower one
                        const bool asc = (((r * kSortThreads) & k) == 0);  // bit k of the element index lies in the register part (k > j >= 1024)
                        const unsigned lo = min(key[r], key[rp]), hi = max(key[r], key[rp]);
                        key[r] = asc ? lo : hi;
                        key[rp] = asc ? hi : lo;
                    }
                }
            } else {
                if (j >= 64) {
                    __syncthreads();  // the previous exchange's reads are done
#pragma unroll
                    for (int r = 0; r < R; r++) keys[r * kSortThreads + tid] = key[r];
                    __syncthreads();
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int i = r * kSortThreads + tid;
                    const unsigned other = j >= 64 ? keys[r * kSortThreads + (tid ^ j)] : (unsigned)__shfl_xor((int)key[r], j, 64);
                    const bool keep_min = ((i & j) == 0) == ((i & k) == 0);
                    key[r] = keep_min ? min(key[r], other) : max(key[r], other);
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < R; r++) keys[r * kSortThreads + tid] = key[r];
    __syncthreads();
    // ids and positions in key order; where a run of equal ids starts, the index one past its end (binary search in the
    // sorted keys), elsewhere -1
    for (int i = threadIdx.x; i < n; i += kSortThreads) {
        const unsigned key = keys[i];
        const bool real = key != 0xffffffffu;
        const unsigned id = key >> shift;
        sorted_ids[i] = real ? (int32_t)id : -1;
        order[i] = (int32_t)(key & ((1u << shift) - 1));
        int end = -1;
        if (real && (i == 0 || (keys[i - 1] >> shift) != id)) {
            int lo = i + 1, hi = n;  // first index in [lo, hi] whose id differs (padding keys count as different)
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                const unsigned km = keys[mid];
                if (km != 0xffffffffu && (km >> shift) == id) lo = mid + 1;
                else hi = mid;
            }
            end = lo;
        }
        run_end[i] = end;
    }
}

// scatter_rows_kernel without the host-built segment table: a wave looks at sorted position k, leaves unless k starts
// a run of equal ids, and adds the run's rows in order.  The hot rows of a Zipf batch are chains of hundreds of
// dependent adds whose speed is set by how many row loads are in flight, so a lane takes only two columns (a wave 128)
// and a long run is walked 64 rows at a time, all 64 loads issued before the first add.
template <typename T> struct Pair;
template <> struct Pair<float> { typedef float2 type; };
template <> struct Pair<bf16_t> { typedef __attribute__((ext_vector_type(2))) __bf16 type; };
template <typename T>
__global__ __launch_bounds__(kThreads) void scatter_runs_kernel(const T* __restrict__ go, float* __restrict__ gw,
                                                                const int32_t* __restrict__ sorted_ids,
                                                                const int32_t* __restrict__ order,
                                                                const int32_t* __restrict__ run_end, int n, int hidden, int slabs) {
    typedef typename Pair<T>::type P2;
    const int lane = threadIdx.x & 63;
    const size_t wave = __builtin_amdgcn_readfirstlane((int)(((size_t)blockIdx.x * kThreads + threadIdx.x) >> 6));
    const int begin = (int)(wave / slabs);
    if (begin >= n) return;
    const int end = run_end[begin];
    if (end < 0) return;  // not the start of a run
    const int row = sorted_ids[begin];
    const int col = ((int)(wave % slabs) * kWave + lane) * 2;
    if (col >= hidden) return;
    float* dst = gw + (size_t)row * hidden + col;
    float2 acc = *reinterpret_cast<const float2*>(dst);
    const T* src = go + col;
    int k = begin;
    for (; k + 64 <= end; k += 64) {
        P2 p[64];
#pragma unroll
        for (int u = 0; u < 64; u++) p[u] = *reinterpret_cast<const P2*>(src + (size_t)order[k + u] * hidden);
#pragma unroll
        for (int u = 0; u < 64; u++) {
            acc.x += (float)p[u][0];
            acc.y += (float)p[u][1];
        }
    }
    for (; k + 8 <= end; k += 8) {
        P2 p[8];
#pragma unroll
        for (int u = 0; u < 8; u++) p[u] = *reinterpret_cast<const P2*>(src + (size_t)order[k + u] * hidden);
#pragma unroll
        for (int u = 0; u < 8; u++) {
            acc.x += (float)p[u][0];
            acc.y += (float)p[u][1];
        }
    }
    for (; k < end; k++) {
        const P2 p = *reinterpret_cast<const P2*>(src + (size_t)order[k] * hidden);
        acc.x += (float)p[0];
        acc.y += (float)p[1];
    }
    *reinterpret_cast<float2*>(dst) = acc;
}

// The device route takes batches whose keys fit 32 bits and whose rows are whole column pairs.
bool scatter_index_on_device(size_t n_ids, size_t vocab, int* n_pow2, int* shift) {
    if (n_ids == 0 || n_ids > (size_t)kSortMax) return false;
    int p = kSortThreads, sh = 10;  // the sort works on whole multiples of its 1024 threads
    while ((size_t)p < n_ids) { p <<= 1; sh++; }
    if ((unsigned long long)vocab << sh >= 0xffffffffull) return false;
    *n_pow2 = p;
    *shift = sh;
    return true;
}
bool scatter_on_device(const void* go, const float* gw, int dtype, size_t n_ids, size_t vocab, size_t hidden, int* n_pow2, int* shift) {
    (void)dtype;
    if (hidden % 2 != 0 || !eisen_aligned(go, 8) || !eisen_aligned(gw, 8)) return false;
    return scatter_index_on_device(n_ids, vocab, n_pow2, shift);
}

// index = [sorted ids | positions in sorted order | run ends], n_ids ints each
void scatter_launch_sort(eisen_ctx* ctx, const int32_t* ids_dev, size_t n_ids, size_t vocab, int n_pow2, int shift, int32_t* index) {
    int32_t* sorted_ids = index;
    int32_t* order = sorted_ids + n_ids;
    int32_t* run_end = order + n_ids;
    switch (n_pow2 / kSortThreads) {
        case 1: scatter_sort_kernel<1><<<1, kSortThreads, 0, ctx->stream>>>(ids_dev, (int)n_ids, shift, (int)vocab, sorted_ids, order, run_end); break;
        case 2: scatter_sort_kernel<2><<<1, kSortThreads, 0, ctx->stream>>>(ids_dev, (int)n_ids, shift, (int)vocab, sorted_ids, order, run_end); break;
        case 4: scatter_sort_kernel<4><<<1, kSortThreads, 0, ctx->stream>>>(ids_dev, (int)n_ids, shift, (int)vocab, sorted_ids, order, run_end); break;
        case 8: scatter_sort_kernel<8><<<1, kSortThreads, 0, ctx->stream>>>(ids_dev, (int)n_ids, shift, (int)vocab, sorted_ids, order, run_end); break;
        default: scatter_sort_kernel<16><<<1, kSortThreads, 0, ctx->stream>>>(ids_dev, (int)n_ids, shift, (int)vocab, sorted_ids, order, run_end); break;
    }
}
void scatter_launch_runs(eisen_ctx* ctx, const int32_t* index, const void* go, float* gw, int dtype, size_t n_ids, size_t hidden) {
    const int32_t* sorted_ids = index;
    const int32_t* order = sorted_ids + n_ids;
    const int32_t* run_end = order + n_ids;
    const int slabs = (int)eisen_ceil_div(hidden, (size_t)kWave * 2);
    const unsigned blocks = (unsigned)eisen_ceil_div(n_ids * slabs, (size_t)(kThreads / kWave));
    if (dtype == EISEN_F32) scatter_runs_kernel<float><<<blocks, kThreads, 0, ctx->stream>>>((const float*)go, gw, sorted_ids, order, run_end, (int)n_ids, (int)hidden, slabs);
    else scatter_runs_kernel<bf16_t><<<blocks, kThreads, 0, ctx->stream>>>((const bf16_t*)go, gw, sorted_ids, order, run_end, (int)n_ids, (int)hidden, slabs);
}

int scatter_device_route(eisen_ctx* ctx, const int32_t* ids_dev, const void* go, float* gw, int dtype, size_t n_ids, size_t vocab, size_t hidden,
                         int n_pow2, int shift) {
    void* dev = nullptr;
    int rc = eisen_hip_malloc(ctx, 3 * n_ids * sizeof(int32_t), &dev);
    if (rc) return rc;
    {
        // algorithmic bytes: every row of dOut read once, every touched row of the f32 gradient read and written once; the
        // touched rows are not known on the host here, so the entry counts dOut and the index only (a lower bound)
        EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "scatter_rows_bf16" : "scatter_rows_f32",
                            (double)n_ids * (double)hidden * eisen_dtype_size(dtype) + 16.0 * (double)n_ids);
        scatter_launch_sort(ctx, ids_dev, n_ids, vocab, n_pow2, shift, (int32_t*)dev);
        scatter_launch_runs(ctx, (const int32_t*)dev, go, gw, dtype, n_ids, hidden);
    }
    hipError_t e = hipGetLastError();
    const int rc_free = eisen_hip_free(ctx, dev);  // stream-ordered: the block is reused only by later work
    if (e != hipSuccess) return eisen_set_error(ctx, (int)e, "scatter kernels: %s", hipGetErrorString(e));
    return rc_free;
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
    int n_pow2 = 0, shift = 0;
    if (scatter_on_device(go, gw, dtype, n_ids, vocab, hidden, &n_pow2, &shift)) {
        // the index is built on the device: the host only hands the ids over
        void* dids = nullptr;
        int rc = eisen_hip_malloc(ctx, n_ids * sizeof(int32_t), &dids);
        if (rc) return rc;
        rc = eisen_hip_htod(ctx, dids, ids_host, n_ids * sizeof(int32_t));
        if (!rc) rc = scatter_device_route(ctx, (const int32_t*)dids, go, gw, dtype, n_ids, vocab, hidden, n_pow2, shift);
        const int rc_free = eisen_hip_free(ctx, dids);
        return rc ? rc : rc_free;
    }
    // larger batches: stable order of positions by token id on the host, ties keep ascending position
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

extern "C" int eisen_hip_gather_backward_dev(eisen_ctx* ctx, const int32_t* ids_dev, const void* go, float* gw, int dtype, size_t n_ids,
                                             size_t vocab, size_t hidden) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ids_dev && go && gw, EISEN_E_ARG, "gather_backward_dev: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "gather_backward_dev: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, vocab > 0 && vocab < (size_t(1) << 31) && hidden > 0 && hidden < (size_t(1) << 30) && n_ids < (size_t(1) << 31),
                  EISEN_E_SHAPE, "gather_backward_dev: sizes out of range");
    if (n_ids == 0) return 0;
    int n_pow2 = 0, shift = 0;
    if (scatter_on_device(go, gw, dtype, n_ids, vocab, hidden, &n_pow2, &shift))
        return scatter_device_route(ctx, ids_dev, go, gw, dtype, n_ids, vocab, hidden, n_pow2, shift);
    // shapes the device route does not take: the ids come back to the host (this synchronises) for the host-built index
    std::vector<int32_t> host(n_ids);
    int rc = eisen_hip_dtoh(ctx, host.data(), ids_dev, n_ids * sizeof(int32_t));
    if (rc) return rc;
    return eisen_hip_gather_backward(ctx, host.data(), go, gw, dtype, n_ids, vocab, hidden);
}

// The two halves of eisen_hip_gather_backward_dev for a caller that knows the ids long before the gradient exists (the token ids
// of a training step are known when its forward pass starts): the index depends on the ids alone.
extern "C" int eisen_hip_gather_index_dev(eisen_ctx* ctx, const int32_t* ids_dev, size_t n_ids, size_t vocab, int32_t* index) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ids_dev && index, EISEN_E_ARG, "gather_index_dev: null pointer");
    EISEN_REQUIRE(ctx, vocab > 0 && vocab < (size_t(1) << 31), EISEN_E_SHAPE, "gather_index_dev: vocab out of range");
    if (n_ids == 0) return 0;
    int n_pow2 = 0, shift = 0;
    EISEN_REQUIRE(ctx, scatter_index_on_device(n_ids, vocab, &n_pow2, &shift), EISEN_E_SHAPE,
                  "gather_index_dev: %zu ids of a vocabulary of %zu are more than the device-side index takes", n_ids, vocab);
    EisenProfScope prof(ctx, "scatter_index", 16.0 * (double)n_ids);
    scatter_launch_sort(ctx, ids_dev, n_ids, vocab, n_pow2, shift, index);
    EISEN_LAUNCH_CHECK(ctx, "scatter_sort_kernel");
    return 0;
}

extern "C" int eisen_hip_gather_backward_indexed(eisen_ctx* ctx, const int32_t* index, const void* go, float* gw, int dtype, size_t n_ids,
                                                 size_t vocab, size_t hidden) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, index && go && gw, EISEN_E_ARG, "gather_backward_indexed: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "gather_backward_indexed: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, vocab > 0 && vocab < (size_t(1) << 31) && hidden > 0 && hidden < (size_t(1) << 30), EISEN_E_SHAPE,
                  "gather_backward_indexed: vocab/hidden out of range");
    if (n_ids == 0) return 0;
    int n_pow2 = 0, shift = 0;
    EISEN_REQUIRE(ctx, scatter_on_device(go, gw, dtype, n_ids, vocab, hidden, &n_pow2, &shift), EISEN_E_SHAPE,
                  "gather_backward_indexed: rows of %zu values at these addresses need eisen_hip_gather_backward_dev", hidden);
    EisenProfScope prof(ctx, dtype == EISEN_BF16 ? "scatter_rows_bf16" : "scatter_rows_f32", (double)n_ids * (double)hidden * eisen_dtype_size(dtype) + 16.0 * (double)n_ids);
    scatter_launch_runs(ctx, index, go, gw, dtype, n_ids, hidden);
    EISEN_LAUNCH_CHECK(ctx, "scatter_runs_kernel");
    return 0;
}
