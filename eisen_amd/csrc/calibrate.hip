// Measured ceilings for the MFMA roofline figures: what this GPU sustains on nothing but v_mfma_f32_32x32x16_bf16, and on
// the same loop with its operands re-read from LDS at the rate of a GEMM's wave tile.  The published peak (2.5 PFLOP/s
// dense bf16) assumes the boost clock; under sustained matrix load the part holds a lower clock, so a kernel's distance
// from what is reachable is better read against these numbers, measured in the same process as the kernel.
// No counterpart in the reference (its kernels use no matrix instructions); a measurement aid, not an operator.
#include "attention_common.cuh"
#include "device_utils.cuh"
#include "runtime.h"

namespace {

// Each wave: four independent 32x32 accumulators (a 64x64 wave tile), 16 MFMAs per iteration = four contraction steps.
// READS: 16-byte LDS operand reads (1 KB per wave instruction) per 16 MFMAs: 0 = operands stay in registers; 16 = the
// 64x64 wave tile of the 8-wave GEMM kernels (two A and two B reads per step); 8 = the ratio of a 128x128 wave tile;
// 24 and 32 = more than any kernel here issues in 16-byte reads (a 64x64 wave tile whose second operand comes through
// 8-byte transposing reads issues 24 read instructions for the same bytes): where the LDS starts to hold the MFMAs back.
// a bf16 with random sign and mantissa and an exponent spread over 2^-4 .. 2^-1: operands whose bits change from one MFMA to
// the next the way those of a trained layer's activations and gradients do
__device__ __forceinline__ bf16_t random_operand(unsigned i) {
    unsigned h = i * 2654435761u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13; h *= 3266489917u; h ^= h >> 16;
    const unsigned short bits = (unsigned short)((h & 0x8000u) | ((123u + ((h >> 7) & 3u)) << 7) | (h & 0x7Fu));
    return __builtin_bit_cast(bf16_t, bits);
}

// RANDOM_DATA: what the operands hold.  The part's clock under matrix load depends on how many operand bits toggle between
// consecutive MFMAs: a GEMM on all-zero or constant matrices runs a third faster than on random ones.  false: a
// few dozen distinct small values (the optimistic ceiling); true: random signs, mantissas and exponents.
template <int READS>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(int iters, float* sink, int random_data) {
    __shared__ __attribute__((aligned(16))) bf16_t tile[16 * 512];  // 16 operand reads' worth of chunks
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16 * 512; i += 512)
        tile[i] = random_data ? random_operand(blockIdx.x * 8192u + i) : (bf16_t)(0.002f * (float)((i * 37) % 113) - 0.11f);
    __syncthreads();
    bf16x8 a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            a[j][e] = random_data ? random_operand(0x10000000u + (blockIdx.x * 512u + threadIdx.x) * 64u + j * 8 + e)
                                  : (bf16_t)(0.003f * (float)((lane * 7 + j * 13 + e * 5) % 61) - 0.09f);
            b[j][e] = random_data ? random_operand(0x20000000u + (blockIdx.x * 512u + threadIdx.x) * 64u + j * 8 + e)
                                  : (bf16_t)(0.004f * (float)((lane * 11 + j * 3 + e * 17) % 53) - 0.10f);
        }
    f32x16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;
    const bf16x8* src = reinterpret_cast<const bf16x8*>(tile) + lane;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            if (READS > 0) {
                constexpr int PER_STEP = READS / 4;  // 2, 4, 6 or 8
                const int base = ((it * 4 + s) * PER_STEP) & 15;
#pragma unroll
                for (int r = 0; r < PER_STEP; r++) {
                    const bf16x8 x = src[((base + r) & 15) * 64];
                    if (r & 1) b[(s + (r >> 1)) & 3] = x;
                    else a[(s + (r >> 1)) & 3] = x;
                    if (r >= 4) asm volatile("" ::"v"(x));  // (a read whose value a later read of the step overwrites is still made)
                }
            }
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], b[s], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], b[(s + 1) & 3], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(s + 1) & 3], b[s], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(s + 1) & 3], b[(s + 1) & 3], acc[3], 0, 0, 0);
        }
    }
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int v = 0; v < 16; v++) t += acc[k][v];
    if (t == 12345.678f) sink[blockIdx.x * 512 + threadIdx.x] = t;  // keeps the loop alive; never true for these operands
}

// A model of the tile loop of the key-stationary attention-backward kernel (attention_bwd.hip), built from the same
// instructions on made-up data, so that each of its parts can be timed alone and together at one or two waves per SIMD:
//   1  the 16 MFMAs of a 32 x 32 x (head_dim 64) tile: two chains of four (S, dP), then four pairs (dV, dK)
//   2  the vector work between them: scale, exp2, product and four packed bf16 conversions per element owned
//   4  the LDS reads: eight 16-byte operand reads, eight broadcast reads of start values, sixteen 8-byte transposing reads
//   8  the eight direct-to-LDS loads of 1 KB that bring a wave's next Q and dO tile (from a 4 MB region that stays in L2)
// Four waves per block with a private two-stage ring each, as in the kernel.
template <int PARTS>
__global__ __launch_bounds__(256, 2) void tile_model_kernel(int iters, const char* gsrc, float* sink) {
    constexpr int STAGE = 8448;
    __shared__ __attribute__((aligned(1024))) char lds[4 * 2 * STAGE];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    char* ring = lds + wave * 2 * STAGE;
    for (int i = lane; i < 2 * STAGE / 4; i += 64) reinterpret_cast<float*>(ring)[i] = 0.001f * (float)((i * 37) % 113) - 0.05f;
    __syncthreads();
    bf16x8 kf[4], vn[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            kf[j][e] = (bf16_t)(0.003f * (float)((lane * 7 + j * 13 + e * 5) % 61) - 0.09f);
            vn[j][e] = (bf16_t)(0.004f * (float)((lane * 11 + j * 3 + e * 17) % 53) - 0.10f);
        }
    f32x16 dk[2], dv[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) { dk[t][v] = 0.f; dv[t][v] = 0.f; }
    // 16 tiles of 8 KB per wave; the blocks of an XCD share one 512 KB set
    const char* gbase = gsrc + (size_t)((blockIdx.x % 8) * 4 + wave) * 16 * 8192;
    const unsigned loff = lane * 16;
    f32x16 s, dp;
#pragma unroll
    for (int v = 0; v < 16; v++) { s[v] = -3.f - 0.01f * v; dp[v] = 0.5f; }
    if (PARTS & 8) {
#pragma unroll
        for (int r = 0; r < 8; r++) load_lds_16(gbase, loff + r * 1024, ring + r * 1024);
    }
    for (int it = 0; it < iters; it++) {
        char* stage = ring + (it & 1) * STAGE;
        if (PARTS & 8) wait_direct_loads();
#pragma unroll
        for (int j = 0; j < 4; j++) asm volatile("" : "+v"(kf[j]), "+v"(vn[j]));  // nothing is hoisted out of the loop
        if (PARTS & 4) {
            const float* st = reinterpret_cast<const float*>(stage + 8192);
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const float4 l4 = *reinterpret_cast<const float4*>(st + 8 * vg + 4 * (lane >> 5));
                const float4 d4 = *reinterpret_cast<const float4*>(st + 32 + 8 * vg + 4 * (lane >> 5));
                s[4 * vg] = l4.x; s[4 * vg + 1] = l4.y; s[4 * vg + 2] = l4.z; s[4 * vg + 3] = l4.w;
                dp[4 * vg] = d4.x; dp[4 * vg + 1] = d4.y; dp[4 * vg + 2] = d4.z; dp[4 * vg + 3] = d4.w;
            }
        }  // without the LDS reads the two score accumulators keep running: no start values to set up, nothing but the MFMAs
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            bf16x8 qa = kf[(ks + 1) & 3], da = vn[(ks + 1) & 3];
            if (PARTS & 4) {
                const int at = (lane & 31) * 128 + ((ks * 2 + (lane >> 5)) ^ (lane & 7)) * 16;  // byte offset, chunks permuted by row
                qa = *reinterpret_cast<const bf16x8*>(stage + at);
                da = *reinterpret_cast<const bf16x8*>(stage + 4096 + at);
            }
            if (PARTS & 1) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vn[ks], dp, 0, 0, 0);
            } else { s[ks] += (float)qa[0]; dp[ks] += (float)da[0]; }
        }
        bf16x8 dotr[2][2], qtr[2][2];
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
                if (PARTS & 4) {
                    const int at = (t * 16 + (lane >> 4) * 2) * 64 + ((dt * 4 + ((lane >> 2) & 3)) ^ (lane & 7)) * 8;  // element offset, rows 0..30
                    const bf16_t* p0 = reinterpret_cast<const bf16_t*>(stage + 4096) + at;
                    const bf16_t* p1 = reinterpret_cast<const bf16_t*>(stage) + at;
                    dotr[dt][t] = concat4(lds_read_tr(p0), lds_read_tr(p0 + 64));
                    qtr[dt][t] = concat4(lds_read_tr(p1), lds_read_tr(p1 + 64));
                } else { dotr[dt][t] = kf[dt * 2 + t]; qtr[dt][t] = vn[dt * 2 + t]; }
            }
        if ((PARTS & 8) && it + 1 < iters) {
            char* nxt = ring + ((it + 1) & 1) * STAGE;
            const char* g = gbase + ((it + 1) & 15) * 8192;
#pragma unroll
            for (int r = 0; r < 8; r++) load_lds_16(g, loff + r * 1024, nxt + r * 1024);
        }
        bf16x8 pf[2], dsf[2];
        if (PARTS & 2) {
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; v++) p[v] = fast_exp2(s[v] * 0.18f);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                pf[v >> 3][v & 7] = (bf16_t)p[v];
                dsf[v >> 3][v & 7] = (bf16_t)(p[v] * dp[v]);
            }
        } else {
            typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int t = 0; t < 2; t++) {
                u32x4 x, y;
#pragma unroll
                for (int e = 0; e < 4; e++) { x[e] = __builtin_bit_cast(unsigned, s[t * 4 + e]); y[e] = __builtin_bit_cast(unsigned, dp[t * 4 + e]); }
                pf[t] = __builtin_bit_cast(bf16x8, x);
                dsf[t] = __builtin_bit_cast(bf16x8, y);
            }
        }
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
                if (PARTS & 1) {
                    dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[t], dotr[dt][t], dv[dt], 0, 0, 0);
                    dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[t], qtr[dt][t], dk[dt], 0, 0, 0);
                } else { dv[dt][t] += (float)pf[t][0] * (float)dotr[dt][t][0]; dk[dt][t] += (float)dsf[t][0] * (float)qtr[dt][t][0]; }
            }
    }
    wait_direct_loads();
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 2; k++)
#pragma unroll
        for (int v = 0; v < 16; v++) t += dk[k][v] + dv[k][v];
    if (t == 12345.678f) sink[blockIdx.x * 256 + threadIdx.x] = t;  // keeps the loop alive; never true for these operands
}


// A model of the tile loop that a one-pass attention backward would have (the score tile and dP computed once, dK, dV and a
// partial dQ from the same pass), on made-up data like the model above, to be set against that model and the two kernels'
// own loops.  A workgroup of four waves owns 128 keys, 32 per wave, and its waves work on the same (query head, 32-query
// tile) item at the same time, so that
//   * the item's Q and dO tile is loaded once per workgroup (two 1 KB direct-to-LDS loads per wave instead of eight),
//   * each wave leaves its dS tile (32 keys x 32 queries, bf16) in LDS, and after the item's one barrier every wave
//     multiplies the four dS tiles by its 16 of the 64 columns of K: eight v_mfma_f32_16x16x32_bf16, the same matrix time
//     as four 32x32x16, and a dQ partial that is complete over the workgroup's 128 keys,
//   * the partial (16 x 32 f32 per wave, 8 KB per workgroup and item) goes to global memory for a later kernel to add
//     up over key chunks in a fixed order (WRITE = false leaves these stores out).
// The dQ product of item t runs behind the barrier of item t + 1, so an item costs one barrier.
template <bool WRITE>
__global__ __launch_bounds__(256, 2) void onepass_tile_model_kernel(int iters, const char* gsrc, char* gdst, float* sink) {
    constexpr int STAGE = 8448, XCH = 4 * 2048;
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE + 2 * XCH];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int i = threadIdx.x; i < (2 * STAGE + 2 * XCH) / 4; i += 256) reinterpret_cast<float*>(lds)[i] = 0.001f * (float)((i * 37) % 113) - 0.05f;
    __syncthreads();
    bf16x8 kf[4], vn[4], ktr[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            kf[j][e] = (bf16_t)(0.003f * (float)((lane * 7 + j * 13 + e * 5) % 61) - 0.09f);
            vn[j][e] = (bf16_t)(0.004f * (float)((lane * 11 + j * 3 + e * 17) % 53) - 0.10f);
            ktr[j][e] = (bf16_t)(0.002f * (float)((lane * 5 + j * 7 + e * 11) % 59) - 0.06f);
        }
    f32x16 dk[2], dv[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) { dk[t][v] = 0.f; dv[t][v] = 0.f; }
    // 16 items of 8 KB per workgroup; the blocks of an XCD share one 512 KB set that stays in its L2
    const char* gbase = gsrc + (size_t)((blockIdx.x % 32) * 16) * 8192;
    // partial dQ: 16 slots of 8 KB per workgroup, written round-robin
    char* dst = gdst + (size_t)blockIdx.x * 16 * 8192;
    const unsigned loff = lane * 16;
    f32x16 s, dp;
    float tail = 0.f;
#pragma unroll
    for (int r = 0; r < 2; r++) load_lds_16(gbase, loff + (wave * 2 + r) * 1024, lds + (wave * 2 + r) * 1024);
    for (int it = 0; it < iters; it++) {
        char* stage = lds + (it & 1) * STAGE;
        char* xch = lds + 2 * STAGE + (it & 1) * XCH;
        const char* xch_prev = lds + 2 * STAGE + ((it & 1) ^ 1) * XCH;
        // this item's tile has landed and the previous item's dS tiles are written: the item's one barrier
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int j = 0; j < 4; j++) asm volatile("" : "+v"(kf[j]), "+v"(vn[j]), "+v"(ktr[j]));  // nothing is hoisted out of the loop
        // the previous item's dQ partial: [16 columns of this wave] x [32 queries], summed over the four waves' key blocks
        {
            f32x4 dq[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int kb = 0; kb < 4; kb++)
#pragma unroll
                for (int nb = 0; nb < 2; nb++) {
                    const int q = nb * 16 + (lane & 15);
                    const bf16x8 ds = *reinterpret_cast<const bf16x8*>(xch_prev + kb * 2048 + q * 64 + (((lane >> 4) ^ (q >> 1)) & 3) * 16);
                    dq[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ktr[kb], ds, dq[nb], 0, 0, 0);
                }
            if (WRITE) {
#pragma unroll
                for (int nb = 0; nb < 2; nb++) {
                    const int q = nb * 16 + (lane & 15);
                    *reinterpret_cast<f32x4*>(dst + (it & 15) * 8192 + q * 256 + (wave * 16 + (lane >> 4) * 4) * 4) = dq[nb];
                }
            } else {
                tail += dq[0][0] + dq[1][3];
            }
        }
        // the next item's tile: this wave's quarter of it
        if (it + 1 < iters) {
            char* nxt = lds + ((it + 1) & 1) * STAGE;
            const char* g = gbase + ((it + 1) & 15) * 8192;
#pragma unroll
            for (int r = 0; r < 2; r++) load_lds_16(g, loff + (wave * 2 + r) * 1024, nxt + (wave * 2 + r) * 1024);
        }
        {
            const float* st = reinterpret_cast<const float*>(stage + 8192);
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const float4 l4 = *reinterpret_cast<const float4*>(st + 8 * vg + 4 * (lane >> 5));
                const float4 d4 = *reinterpret_cast<const float4*>(st + 32 + 8 * vg + 4 * (lane >> 5));
                s[4 * vg] = l4.x; s[4 * vg + 1] = l4.y; s[4 * vg + 2] = l4.z; s[4 * vg + 3] = l4.w;
                dp[4 * vg] = d4.x; dp[4 * vg + 1] = d4.y; dp[4 * vg + 2] = d4.z; dp[4 * vg + 3] = d4.w;
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int at = (lane & 31) * 128 + ((ks * 2 + (lane >> 5)) ^ (lane & 7)) * 16;
            const bf16x8 qa = *reinterpret_cast<const bf16x8*>(stage + at);
            const bf16x8 da = *reinterpret_cast<const bf16x8*>(stage + 4096 + at);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[ks], s, 0, 0, 0);
            dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vn[ks], dp, 0, 0, 0);
        }
        bf16x8 dotr[2][2], qtr[2][2];
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int at = (t * 16 + (lane >> 4) * 2) * 64 + ((dt * 4 + ((lane >> 2) & 3)) ^ (lane & 7)) * 8;
                const bf16_t* p0 = reinterpret_cast<const bf16_t*>(stage + 4096) + at;
                const bf16_t* p1 = reinterpret_cast<const bf16_t*>(stage) + at;
                dotr[dt][t] = concat4(lds_read_tr(p0), lds_read_tr(p0 + 64));
                qtr[dt][t] = concat4(lds_read_tr(p1), lds_read_tr(p1 + 64));
            }
        bf16x8 pf[2], dsf[2];
        {
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; v++) p[v] = fast_exp2(s[v] * 0.18f);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                pf[v >> 3][v & 7] = (bf16_t)p[v];
                dsf[v >> 3][v & 7] = (bf16_t)(p[v] * dp[v]);
            }
        }
        // this wave's dS tile for the other waves: a lane owns query (lane & 31) and, per group of eight keys, four of them
        {
            const int q = lane & 31;
            typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const u64x2 two = __builtin_bit_cast(u64x2, dsf[t]);
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int i = t * 2 + h;
                    *reinterpret_cast<unsigned long long*>(xch + wave * 2048 + q * 64 + ((i ^ (q >> 1)) & 3) * 16 + 8 * (lane >> 5)) = two[h];
                }
            }
        }
#pragma unroll
        for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int t = 0; t < 2; t++) {
                dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[t], dotr[dt][t], dv[dt], 0, 0, 0);
                dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[t], qtr[dt][t], dk[dt], 0, 0, 0);
            }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float t = tail;
#pragma unroll
    for (int k = 0; k < 2; k++)
#pragma unroll
        for (int v = 0; v < 16; v++) t += dk[k][v] + dv[k][v];
    if (t == 12345.678f) sink[blockIdx.x * 256 + threadIdx.x] = t;  // keeps the loop alive; never true for these operands
}

// The two small kernels a one-pass backward needs around its main kernel, for their durations.
// D[row] = sum over 64 columns of dO o O (bf16 rows): a lane takes 8 columns, 8 lanes a row.
__global__ __launch_bounds__(256) void rowdot_model_kernel(const bf16x8* __restrict__ a, const bf16x8* __restrict__ b, float* __restrict__ d, size_t rows) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    float acc = 0.f;
    if (i < rows * 8) {
        const bf16x8 x = a[i], y = b[i];
#pragma unroll
        for (int e = 0; e < 8; e++) acc += (float)x[e] * (float)y[e];
    }
    acc += __shfl_xor(acc, 1);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 4);
    if (i < rows * 8 && (threadIdx.x & 7) == 0) d[i >> 3] = acc;
}
// dQ[row] = the sum, in plane order, of the f32 partials of the key chunks a causal query at position row % seq sees
// (position / chunk + 1 of them), stored as bf16; a lane takes 8 of a row's 64 columns.
__global__ __launch_bounds__(256) void partial_sum_model_kernel(const float* __restrict__ part, bf16x8* __restrict__ out, size_t rows, int seq, int chunk) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * 8) return;
    const int planes = (int)((i >> 3) % (size_t)seq) / chunk + 1;
    f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
    for (int p = 0; p < planes; p++) {
        const f32x4* src = reinterpret_cast<const f32x4*>(part + (size_t)p * rows * 64) + i * 2;
        lo += __builtin_nontemporal_load(src);
        hi += __builtin_nontemporal_load(src + 1);
    }
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 4; e++) { o[e] = (bf16_t)lo[e]; o[4 + e] = (bf16_t)hi[e]; }
    out[i] = o;
}

}  // namespace

static int mfma_ceiling_run(eisen_ctx* ctx, int lds_reads_per_16_mfma, int random_data, int iters, double* tflops_out);
extern "C" int eisen_hip_mfma_ceiling(eisen_ctx* ctx, int lds_reads_per_16_mfma, int iters, double* tflops_out) {
    return mfma_ceiling_run(ctx, lds_reads_per_16_mfma, 0, iters, tflops_out);
}
extern "C" int eisen_hip_mfma_ceiling_random(eisen_ctx* ctx, int lds_reads_per_16_mfma, int iters, double* tflops_out) {
    return mfma_ceiling_run(ctx, lds_reads_per_16_mfma, 1, iters, tflops_out);
}
static int mfma_ceiling_run(eisen_ctx* ctx, int lds_reads_per_16_mfma, int random_data, int iters, double* tflops_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, tflops_out != nullptr, EISEN_E_ARG, "mfma_ceiling: tflops_out is null");
    EISEN_REQUIRE(ctx, lds_reads_per_16_mfma == 0 || lds_reads_per_16_mfma == 8 || lds_reads_per_16_mfma == 16 || lds_reads_per_16_mfma == 24 || lds_reads_per_16_mfma == 32, EISEN_E_ARG,
                  "mfma_ceiling: lds_reads_per_16_mfma must be 0, 8, 16, 24 or 32, got %d", lds_reads_per_16_mfma);
    EISEN_REQUIRE(ctx, iters > 0 && iters <= (1 << 20), EISEN_E_ARG, "mfma_ceiling: iters %d outside (0, 2^20]", iters);
    hipDeviceProp_t prop;
    EISEN_HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const int blocks = prop.multiProcessorCount;  // one 8-wave workgroup per CU: two waves per SIMD
    void* sink = nullptr;
    int rc = eisen_workspace(ctx, (size_t)blocks * 512 * sizeof(float), &sink);
    if (rc) return rc;
    hipEvent_t e0, e1;
    EISEN_HIP_TRY(ctx, hipEventCreate(&e0));
    EISEN_HIP_TRY(ctx, hipEventCreate(&e1));
    auto launch = [&](int n) {
        if (lds_reads_per_16_mfma == 0) mfma_ceiling_kernel<0><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink, random_data);
        else if (lds_reads_per_16_mfma == 8) mfma_ceiling_kernel<8><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink, random_data);
        else if (lds_reads_per_16_mfma == 16) mfma_ceiling_kernel<16><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink, random_data);
        else if (lds_reads_per_16_mfma == 24) mfma_ceiling_kernel<24><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink, random_data);
        else mfma_ceiling_kernel<32><<<blocks, 512, 0, ctx->stream>>>(n, (float*)sink, random_data);
    };
    launch(iters);  // warm-up: clocks and code object
    hipError_t err = hipEventRecord(e0, ctx->stream);
    launch(iters);
    if (err == hipSuccess) err = hipGetLastError();
    if (err == hipSuccess) err = hipEventRecord(e1, ctx->stream);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return eisen_set_error(ctx, (int)err, "mfma_ceiling: %s", hipGetErrorString(err));
    const double flops = (double)blocks * 8.0 * (double)iters * 16.0 * 32768.0;  // waves x iterations x MFMAs x flop per MFMA
    *tflops_out = ms > 0.f ? flops / (ms * 1e-3) / 1e12 : 0.0;
    return 0;
}

extern "C" int eisen_hip_attention_tile_model(eisen_ctx* ctx, int parts, int waves_per_simd, int iters, double* ns_per_tile_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ns_per_tile_out != nullptr, EISEN_E_ARG, "attention_tile_model: ns_per_tile_out is null");
    EISEN_REQUIRE(ctx, parts == 1 || parts == 3 || parts == 7 || parts == 8 || parts == 15 || parts == 16 || parts == 32, EISEN_E_ARG,
                  "attention_tile_model: parts must be 1, 3, 7, 8, 15, 16 or 32, got %d", parts);
    EISEN_REQUIRE(ctx, waves_per_simd == 1 || waves_per_simd == 2, EISEN_E_ARG, "attention_tile_model: waves_per_simd must be 1 or 2, got %d", waves_per_simd);
    EISEN_REQUIRE(ctx, iters > 0 && iters <= (1 << 20), EISEN_E_ARG, "attention_tile_model: iters %d outside (0, 2^20]", iters);
    hipDeviceProp_t prop;
    EISEN_HIP_TRY(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const int blocks = prop.multiProcessorCount * waves_per_simd;  // four waves per block, one per SIMD
    const size_t src_bytes = (size_t)8 * 4 * 16 * 8192, sink_bytes = (size_t)blocks * 256 * sizeof(float);
    const size_t dst_bytes = parts == 16 ? (size_t)blocks * 16 * 8192 : 0;  // the one-pass model's dQ partials
    void* ws = nullptr;
    int rc = eisen_workspace(ctx, src_bytes + sink_bytes + dst_bytes, &ws);
    if (rc) return rc;
    char* src = static_cast<char*>(ws);
    float* sink = reinterpret_cast<float*>(src + src_bytes);
    char* dst = src + src_bytes + sink_bytes;
    rc = eisen_hip_fill(ctx, src, EISEN_F32, 0.f, src_bytes / sizeof(float));
    if (rc) return rc;
    hipEvent_t e0, e1;
    EISEN_HIP_TRY(ctx, hipEventCreate(&e0));
    EISEN_HIP_TRY(ctx, hipEventCreate(&e1));
    auto launch = [&](int n) {
        switch (parts) {
            case 1: tile_model_kernel<1><<<blocks, 256, 0, ctx->stream>>>(n, src, sink); break;
            case 3: tile_model_kernel<3><<<blocks, 256, 0, ctx->stream>>>(n, src, sink); break;
            case 7: tile_model_kernel<7><<<blocks, 256, 0, ctx->stream>>>(n, src, sink); break;
            case 8: tile_model_kernel<8><<<blocks, 256, 0, ctx->stream>>>(n, src, sink); break;
            case 16: onepass_tile_model_kernel<true><<<blocks, 256, 0, ctx->stream>>>(n, src, dst, sink); break;
            case 32: onepass_tile_model_kernel<false><<<blocks, 256, 0, ctx->stream>>>(n, src, dst, sink); break;
            default: tile_model_kernel<15><<<blocks, 256, 0, ctx->stream>>>(n, src, sink); break;
        }
    };
    launch(iters / 8 + 1);  // warm-up: clocks, code object, the source region into the L2
    hipError_t err = hipEventRecord(e0, ctx->stream);
    launch(iters);
    if (err == hipSuccess) err = hipGetLastError();
    if (err == hipSuccess) err = hipEventRecord(e1, ctx->stream);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return eisen_set_error(ctx, (int)err, "attention_tile_model: %s", hipGetErrorString(err));
    *ns_per_tile_out = (double)ms * 1e6 / (double)iters / (double)waves_per_simd;  // a SIMD finishes waves_per_simd tiles per iteration
    return 0;
}

extern "C" int eisen_hip_attention_onepass_parts(eisen_ctx* ctx, size_t rows, int seq, int chunk, double* rowdot_us_out, double* partial_sum_us_out) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, rowdot_us_out != nullptr && partial_sum_us_out != nullptr, EISEN_E_ARG, "attention_onepass_parts: null result pointer");
    EISEN_REQUIRE(ctx, rows > 0 && rows <= (size_t(1) << 22) && seq > 0 && chunk > 0 && seq % chunk == 0 && seq / chunk <= 16 && rows % (size_t)seq == 0, EISEN_E_SHAPE,
                  "attention_onepass_parts: rows %zu (at most 2^22, whole sequences), seq %d, chunk %d (a divisor of seq, at most 16 chunks)", rows, seq, chunk);
    const int planes = seq / chunk;
    const size_t row_bytes = 64 * sizeof(bf16_t), plane_bytes = rows * 64 * sizeof(float);
    void *a = nullptr, *b = nullptr, *d = nullptr, *part = nullptr, *out = nullptr;
    int rc = eisen_hip_malloc(ctx, rows * row_bytes, &a);
    if (!rc) rc = eisen_hip_malloc(ctx, rows * row_bytes, &b);
    if (!rc) rc = eisen_hip_malloc(ctx, rows * sizeof(float), &d);
    if (!rc) rc = eisen_hip_malloc(ctx, plane_bytes * planes, &part);
    if (!rc) rc = eisen_hip_malloc(ctx, rows * row_bytes, &out);
    if (!rc) rc = eisen_hip_fill(ctx, a, EISEN_BF16, 0.5f, rows * 64);
    if (!rc) rc = eisen_hip_fill(ctx, b, EISEN_BF16, 0.25f, rows * 64);
    if (!rc) rc = eisen_hip_fill(ctx, part, EISEN_F32, 0.125f, rows * 64 * (size_t)planes);
    hipEvent_t e[3] = {nullptr, nullptr, nullptr};
    hipError_t err = hipSuccess;
    if (!rc) {
        for (int i = 0; i < 3 && err == hipSuccess; i++) err = hipEventCreate(&e[i]);
        const unsigned blocks = (unsigned)eisen_ceil_div(rows * 8, (size_t)256);
        constexpr int REPS = 10;
        for (int rep = 0; rep < REPS + 1 && err == hipSuccess; rep++) {  // the first round warms up
            if (rep == 1) err = hipEventRecord(e[0], ctx->stream);
            rowdot_model_kernel<<<blocks, 256, 0, ctx->stream>>>(static_cast<const bf16x8*>(a), static_cast<const bf16x8*>(b), static_cast<float*>(d), rows);
        }
        if (err == hipSuccess) err = hipEventRecord(e[1], ctx->stream);
        for (int rep = 0; rep < REPS && err == hipSuccess; rep++)
            partial_sum_model_kernel<<<blocks, 256, 0, ctx->stream>>>(static_cast<const float*>(part), static_cast<bf16x8*>(out), rows, seq, chunk);
        if (err == hipSuccess) err = hipEventRecord(e[2], ctx->stream);
        if (err == hipSuccess) err = hipGetLastError();
        if (err == hipSuccess) err = hipEventSynchronize(e[2]);
        float ms0 = 0.f, ms1 = 0.f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms0, e[0], e[1]);
        if (err == hipSuccess) err = hipEventElapsedTime(&ms1, e[1], e[2]);
        *rowdot_us_out = (double)ms0 * 1e3 / REPS;
        *partial_sum_us_out = (double)ms1 * 1e3 / REPS;
        for (int i = 0; i < 3; i++)
            if (e[i]) (void)hipEventDestroy(e[i]);
    }
    for (void* p : {a, b, d, part, out})
        if (p) (void)eisen_hip_free(ctx, p);
    if (rc) return rc;
    if (err != hipSuccess) return eisen_set_error(ctx, (int)err, "attention_onepass_parts: %s", hipGetErrorString(err));
    return 0;
}
