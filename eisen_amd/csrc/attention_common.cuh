// Shared by the attention kernels (attention.hip: forward, dQ, f32 path and the entry points; attention_bwd.hip: the
// key-stationary dK/dV kernel): launch arguments, MFMA accumulator indexing, LDS tile layouts and loaders.
#pragma once
#include <type_traits>

#include "device_utils.cuh"
#include "runtime.h"

struct AttnArgs {
    const void *Q, *K, *V, *O, *dO;
    void *Out, *dQ, *dK, *dV;
    float *LSE, *D;
    float* L2;  // backward only: -LSE / scale per (batch, query head, position), written by the dQ kernel next to D
    int B, S, Hq, Hkv, G, hd;
    long long q_sb, q_ss, q_sh;
    long long k_sb, k_ss, k_sh;
    float scale, scale_log2e;
    int causal;
    int paired;  // query-stationary kernels: a block runs a long query block and its short mirror image
    // backward only: when set ([S][hd/2] cos/sin), Q and K are rotary-embedded projections and dQ, dK are the
    // gradients of the projections before the rotation (the inverse rotation is applied as the gradients are stored)
    const float2* rope;
    // measurement only (eisen_hip_attention_ablation): which part of the backward kernels' tile loop is left out, 0 = none
    int ablation;
    // measurement only (eisen_hip_attention_timeline): where the kernels drop time stamps of their waves' progress,
    // [kernel][wave][8 stamps][100 MHz counter | shader clock]; waves from stamp_waves on drop none
    long long* stamps;
    int stamp_waves;
};

// Parts of a backward kernel's tile loop that an ablation run leaves out (the results are then wrong by construction; every
// memory access that remains is one the full kernel makes as well).  What a run without one part gains is that part's
// share of the kernel's critical path.
enum AttnAblation {
    kAblNone = 0,
    kAblTransposedReads = 1,  // the LDS transpose reads (operands of the second MFMA group) -> registers already held
    kAblOperandReads = 2,     // the 16-byte LDS operand reads of the score MFMAs -> registers already held
    kAblSecondMfmas = 3,      // the MFMAs after the softmax (dK/dV kernel: dV and dK; dQ kernel: dQ)
    kAblTileLoads = 4,        // the direct-to-LDS loads of every tile after the first
    kAblSoftmax = 5,          // scale, exp2 and the dS product (the bf16 conversions stay)
    kAblScoreMfmas = 6,       // the S and dP MFMAs
    kAblCount = 7,
    kAblTimeline = 7          // nothing left out: the kernels as they are, plus the time stamps of AttnArgs::stamps
};
// Stamps of a wave: 0 kernel entered, 1 / 2 first tile loop begins / ends, 3 its results stored, 4 / 5 second tile loop
// (the mirror block of a pair) begins / ends, 6 its results stored.  Kernel index: 0 forward, 1 dQ, 2 dK/dV.
enum AttnStamp { kStampStart = 0, kStampLoop = 1, kStampLoopEnd = 2, kStampStored = 3, kStampsPerPass = 3 };

// the key-stationary dK / dV kernel for head_dim 32 and 64 (attention_bwd.hip); a.D and a.L2 must have been written
bool eisen_attention_dkv32_supports(const AttnArgs& a);
void eisen_attention_launch_dkv32(eisen_ctx* ctx, const AttnArgs& a);

namespace {


template <bool ON>
__device__ __forceinline__ void attn_stamp(const AttnArgs& a, int kernel, int k, int lane, int wave) {
    if (!ON) return;
    const long long w = wall_clock64(), c = clock64();
    const int id = (int)blockIdx.x * 4 + wave;
    if (lane == 0 && id < a.stamp_waves) {
        long long* p = a.stamps + ((size_t)kernel * a.stamp_waves + id) * 16 + 2 * k;
        p[0] = w;
        p[1] = c;
    }
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef bf16x4 __attribute__((address_space(3))) * lds_bf16x4_ptr;

// 4 consecutive rows of a column out of a row-major LDS tile: within each group of 16 lanes,
// lane i receives rows r0..r0+3 of column c0+i when lane L passes &tile[r0 + L/4][c0 + 4*(L%4)].
__device__ __forceinline__ bf16x4 lds_read_tr(const bf16_t* p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p));
}
__device__ __forceinline__ bf16x8 concat4(bf16x4 lo, bf16x4 hi) {
    bf16x8 r;
    r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
    r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
    return r;
}
// Row index inside a 32x32 MFMA accumulator tile held by register v of a lane in half g.
__device__ __forceinline__ int acc_row(int v, int g) { return 8 * (v >> 2) + 4 * g + (v & 3); }

// Backward of the rotary embedding on NP interleaved pairs: dx0 = g0 c + g1 s, dx1 = -g0 s + g1 c
// (src/graph/ops/transform.rs:592-595); cs points at the (cos, sin) of the first pair.
template <int NP>
__device__ __forceinline__ void unrotate_pairs(float* x, const float2* cs) {
#pragma unroll
    for (int j = 0; j < NP; j++) {
        const float2 t = cs[j];
        const float g0 = x[2 * j], g1 = x[2 * j + 1];
        x[2 * j] = g0 * t.x + g1 * t.y;
        x[2 * j + 1] = -g0 * t.y + g1 * t.x;
    }
}

// K-operand (8 values along the contraction) for contraction step t of a [32-row k-dim] x
// [32-col] block of a row-major LDS tile, in the order the accumulator registers 8t..8t+7 use.
__device__ __forceinline__ bf16x8 lds_tr_operand(const bf16_t* tile, int pitch, int row0, int col0, int t, int lane) {
    const int g = lane >> 5, L = lane & 15, half = (lane >> 4) & 1;
    const bf16_t* p = tile + (row0 + 16 * t + 4 * g + (L >> 2)) * pitch + col0 + 16 * half + 4 * (L & 3);
    return concat4(lds_read_tr(p), lds_read_tr(p + 8 * pitch));
}

// 2^x as the bare hardware instruction: results below 2^-126 flush to zero, which is what a softmax
// weight that small should be; the library exp2f spends four more instructions per value on them.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// A ROWS x HD bf16 tile on its way from a strided global tensor into LDS, held in registers in
// between so the global loads of tile i+1 are in flight while tile i is being used.
template <int HD, int ROWS, int THREADS>
struct TilePrefetch {
    static constexpr int PITCH = HD + 8, CPR = HD / 8, TOTAL = ROWS * CPR;
    static constexpr int CH = (TOTAL + THREADS - 1) / THREADS;
    bf16x8 r[CH];
    __device__ __forceinline__ void fetch(const bf16_t* src, long long row_stride, int first_row, int limit_rows) {
        const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if (first_row + ROWS <= limit_rows) {  // whole tile in range (uniform): plain loads, no selects
#pragma unroll
            for (int i = 0; i < CH; i++) {
                const int c = i * THREADS + threadIdx.x;
                if (TOTAL % THREADS == 0 || c < TOTAL)
                    r[i] = *reinterpret_cast<const bf16x8*>(src + (long long)(first_row + c / CPR) * row_stride + (c % CPR) * 8);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int c = i * THREADS + threadIdx.x;
            const int row = c / CPR, cc = c % CPR, gr = first_row + row;
            r[i] = (c < TOTAL && gr < limit_rows) ? *reinterpret_cast<const bf16x8*>(src + (long long)gr * row_stride + cc * 8) : zero8;
        }
    }
    __device__ __forceinline__ void commit(bf16_t* dst) const {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int c = i * THREADS + threadIdx.x;
            if (c < TOTAL) *reinterpret_cast<bf16x8*>(dst + (c / CPR) * PITCH + (c % CPR) * 8) = r[i];
        }
    }
};

// ---- tiles loaded straight into LDS ----------------------------------------------------------
// Unpadded rows of HD bf16 with permuted chunks (lds_swz in device_utils.cuh).
template <int HD>
__device__ __forceinline__ int tile_swz(int row) { return lds_swz<HD * 2>(row); }
template <int HD>
__device__ __forceinline__ int tile_at(int row, int col) {
    return row * HD + ((((col >> 3) ^ tile_swz<HD>(row)) << 3) | (col & 7));
}
// lds_tr_operand for a swizzled tile
template <int HD>
__device__ __forceinline__ bf16x8 lds_tr_operand_swz(const bf16_t* tile, int row0, int col0, int t, int lane) {
    const int g = lane >> 5, L = lane & 15, half = (lane >> 4) & 1;
    const int row = row0 + 16 * t + 4 * g + (L >> 2), col = col0 + 16 * half + 4 * (L & 3);
    return concat4(lds_read_tr(tile + tile_at<HD>(row, col)), lds_read_tr(tile + tile_at<HD>(row + 8, col)));
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;

// A ROWS x HD bf16 tile of a strided global tensor, loaded into a swizzled LDS tile by WAVES waves with
// no registers in between.  Each wave instruction moves 1 KB (512 / HD rows).  Rows past `limit_rows`
// re-read the last valid row: the kernels mask or zero-weight them, they only have to be finite.
// The loads are asynchronous: wait_direct_loads() before the barrier that publishes the tile.
template <int HD, int ROWS, int WAVES>
struct DirectTile {
    static constexpr int CPR = HD / 8, RPB = 64 / CPR, BLOCKS = ROWS / RPB, PER_WAVE = BLOCKS / WAVES;
    static_assert(ROWS % RPB == 0 && BLOCKS % WAVES == 0, "tile does not split into whole wave loads");
    unsigned off[PER_WAVE];  // byte offset of this lane's chunk from the tile's first row (loop-invariant)
    __device__ __forceinline__ static int lane_row(int wave, int i, int lane) { return (wave * PER_WAVE + i) * RPB + lane / CPR; }
    __device__ __forceinline__ static int lane_chunk(int row, int lane) { return (lane % CPR) ^ tile_swz<HD>(row); }
    __device__ __forceinline__ void init(long long row_stride, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            const int row = lane_row(wave, i, lane);
            off[i] = (unsigned)((row * row_stride + lane_chunk(row, lane) * 8) * 2);
        }
    }
    __device__ __forceinline__ void load(const bf16_t* src, long long row_stride, int first_row, int limit_rows, bf16_t* lds_tile,
                                         int wave, int lane) const {
        if (first_row + ROWS <= limit_rows) {  // whole tile in range (uniform)
            const char* base = reinterpret_cast<const char*>(src + (long long)first_row * row_stride);
#pragma unroll
            for (int i = 0; i < PER_WAVE; i++)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(base + off[i]), (lds_void_ptr)(lds_tile + (wave * PER_WAVE + i) * 512), 16, 0, 0);
            return;
        }
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) {
            const int row = lane_row(wave, i, lane);
            const int gr = min(first_row + row, limit_rows - 1);
            __builtin_amdgcn_global_load_lds((global_void_ptr)(src + (long long)gr * row_stride + lane_chunk(row, lane) * 8),
                                             (lds_void_ptr)(lds_tile + (wave * PER_WAVE + i) * 512), 16, 0, 0);
        }
    }
    // the same tile through load_lds_16 (see there); src + first_row * row_stride must be wave-uniform
    __device__ __forceinline__ void load_untracked(const bf16_t* src, long long row_stride, int first_row, int limit_rows, bf16_t* lds_tile,
                                                   int wave, int lane) const;
};
__device__ __forceinline__ void wait_direct_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// One wave instruction of a direct-to-LDS load, written out: lane l's 16 (4) bytes land at lds_dst + 16 (4) * l.  The
// compiler does not know that these write LDS, so it orders nothing around them: the kernel waits (s_waitcnt vmcnt)
// before it reads what they bring and does not overwrite what is still being read.  With the builtin, the compiler may
// place a wait for every load in flight in front of the next LDS read, the prefetched tile's included.
//   *_saddr: wave-uniform 64-bit base and a 32-bit byte offset per lane (two scalar instructions and the load; no address
//   arithmetic in vector registers); *_vaddr: a 64-bit address per lane.
__device__ __forceinline__ void load_lds_16(const void* base, unsigned lane_offset, const void* lds_dst) {
    const unsigned lds_addr = (unsigned)(size_t)(lds_void_ptr)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_offset), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void load_lds_4(const void* base, unsigned lane_offset, const void* lds_dst) {
    const unsigned lds_addr = (unsigned)(size_t)(lds_void_ptr)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(lane_offset), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void load_lds_16_vaddr(const void* lane_ptr, const void* lds_dst) {
    const unsigned lds_addr = (unsigned)(size_t)(lds_void_ptr)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(lane_ptr) : "memory", "m0");
}

template <int HD, int ROWS, int WAVES>
__device__ __forceinline__ void DirectTile<HD, ROWS, WAVES>::load_untracked(const bf16_t* src, long long row_stride, int first_row, int limit_rows,
                                                                            bf16_t* lds_tile, int wave, int lane) const {
    if (first_row + ROWS <= limit_rows) {  // whole tile in range (uniform)
        const char* base = reinterpret_cast<const char*>(src + (long long)first_row * row_stride);
#pragma unroll
        for (int i = 0; i < PER_WAVE; i++) load_lds_16(base, off[i], lds_tile + (wave * PER_WAVE + i) * 512);
        return;
    }
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {
        const int row = lane_row(wave, i, lane);
        const int gr = min(first_row + row, limit_rows - 1);
        load_lds_16_vaddr(src + (long long)gr * row_stride + lane_chunk(row, lane) * 8, lds_tile + (wave * PER_WAVE + i) * 512);
    }
}

}  // namespace
