// Pieces shared by the GEMM kernels of gemm.hip and gemm_wide.hip: the launch argument block, the operand tiles
// filled by direct-to-LDS loads, and the epilogue that stores a wave's accumulators.
#pragma once
#include <type_traits>
#include <utility>

#include "device_utils.cuh"
#include "runtime.h"

constexpr int kMaxGroup = 8;  // products of one grouped launch
struct GemmArgs {
    const void* A;
    const void* B;
    void* C;
    int M, N, K;
    int lda, ldb, ldc;                 // leading dimensions in elements
    long long sA, sB, sC;              // batch strides in elements
    int accumulate;
    const void* R;                     // optional residual with C's layout: C = R + A*B (accumulate must be 0)
    int split;                         // > 1: K is cut into this many parts; part p > 0 assigns into partial[p-1]
    int k_part;                        // contraction length of one part (a multiple of the slab)
    float* partial;                    // [batch][split-1][M][N] f32, summed into C by a second kernel
    // SwiGLU-backward epilogue (gate != nullptr): the product is dH, the gradient of h = silu(gate) * up; C receives
    // dgate = dH * up * silu'(gate) and C2 receives dup = dH * silu(gate) (all with C's layout, no accumulation, no split-K)
    const void* gate;
    const void* up;
    void* C2;
    // Grouped launch (direct kernel, ngroup > 0): blockIdx.x enumerates the tiles of up to kMaxGroup products that share M, K
    // and the operand orders but have their own A, B, C and N; grp_tile_end[p] = number of tiles of products 0..p
    int ngroup;
    const void* grp_A[kMaxGroup];
    const void* grp_B[kMaxGroup];
    void* grp_C[kMaxGroup];
    int grp_N[kMaxGroup];
    int grp_tile_end[kMaxGroup];
    long long grp_partial_off[kMaxGroup];  // grouped launch with split > 1: where product p's partial results start inside `partial`
    int tile_group;                    // direct kernel: > 0 = N tiles per group of the tile order (see the kernel), 0 = row-major order, < 0 = blocks per XCD
    int vec_c;                         // C rows are 16-byte aligned at every 8th column: the epilogue may use 16-byte accesses
    // K made of up to three segments with their own operands, C (+)= sum_s op(A_s) op(B_s): segment 0 is A/B/lda/ldb,
    // seg_end[s] is the contraction offset at which segment s ends (multiples of 64); nseg <= 1 means plain
    int nseg;
    const void* A_seg[2];
    const void* B_seg[2];
    int lda_seg[2], ldb_seg[2];
    int seg_end[2];
    // Rotary-embedding epilogue (rope != nullptr; bf16 C, whole tiles, no accumulation, residual or split): the batch members
    // below rope_members leave as rope(A*B), row m at position m % rope_seq, heads of rope_head_dim columns (a multiple of 8)
    const float2* rope;                // cos/sin table [>= rope_seq][rope_head_dim / 2]
    int rope_seq, rope_head_dim, rope_members;
};

// gemm_wide.hip: 256 x 256 tiles, four waves of 128 x 128 (plain products, whole tiles only)
bool eisen_gemm_wide_supports(const GemmArgs& g, bool a_kc, bool b_kc, int batch, int dtype_c);
void eisen_gemm_launch_wide(eisen_ctx* ctx, const GemmArgs& g, bool a_kc, bool b_kc, int dtype_c);

// One launch of gemm_wide.hip's kernel over any number of products whose contraction is stored in several pieces:
// C_p (+)= sum_s A_ps^T B_ps with A_ps bf16 [seg_k][M_p], B_ps bf16 [seg_k][N_p], C_p f32 [M_p][N_p] (the weight gradients
// of the Linear layers of a model over several micro-batches, each micro-batch's activations and output gradients where
// its forward and backward pass left them).  The products are described by a table in device memory.
constexpr int kMaxWindowSegments = 8;
struct WideWindowRow {
    int M, N;
    int tile_end;  // number of 256 x 256 tiles of products 0..p
    int pad;
    void* C;
    const void* A[kMaxWindowSegments];  // entries from nseg on repeat the last piece
    const void* B[kMaxWindowSegments];
};
struct WideWindow {
    int nprod, nseg;
    int seg_slabs;  // 32-deep slabs per piece, a multiple of 4
    int accumulate;
    const WideWindowRow* rows;  // device memory, nprod entries
    // Optional meeting point for the workgroups an XCD runs at one time (null: none).  One counter per XCD and group of 32
    // consecutive tiles of its range, zero at launch.  A workgroup counts itself in and waits until its group is complete or
    // `meet_ticks` of the 100 MHz clock have passed, whichever comes first: the wait only keeps the group's tiles close enough
    // in time to share their operand panels in the L2, and no result depends on it.
    int* meet;
    int meet_ticks;
};
// the host's copy of the table: shapes the kernel takes?
bool eisen_gemm_wide_window_supports(const WideWindow& w, const WideWindowRow* host_rows);
void eisen_gemm_launch_wide_window(eisen_ctx* ctx, const WideWindow& w, unsigned tiles);

namespace {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a constant expression
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}


typedef bf16x4 __attribute__((address_space(3))) * lds_bf16x4_ptr;

// Tile (mt, nt) of workgroup `lin` in an order that keeps the tiles an XCD works on at one time (a contiguous range of
// the order, see xcd_contiguous_id; about one tile per CU, 32 per XCD) inside a block of BMT x BNT tiles, which share
// BMT + BNT operand panels in that XCD's L2.  Block rows of BMT tile rows, blocks left to right, row-major inside a
// block; the last block of a row and the last row of blocks may be smaller.
template <int BMT, int BNT>
__device__ __forceinline__ void xcd_block_tile(int lin, int m_tiles, int n_tiles, int& mt, int& nt) {
    lin = xcd_contiguous_id(lin, m_tiles * n_tiles);
    const int row_block = BMT * n_tiles, bi = lin / row_block, rem = lin % row_block;
    const int h = min(BMT, m_tiles - BMT * bi);
    const int bj = rem / (h * BNT), rem2 = rem % (h * BNT);
    const int wdt = min(BNT, n_tiles - BNT * bj);
    mt = BMT * bi + rem2 / wdt;
    nt = BNT * bj + rem2 % wdt;
}

// d(silu(gate) * up) for one element, given dh (src/graph/ops/elementwise.rs:442-455 for silu, :294-331 for mul)
__device__ __forceinline__ void swiglu_backward_elem(float gate, float up, float dh, float& dgate, float& dup) {
    // v_rcp_f32 (1 ulp) instead of the correctly rounded division's ten instructions: in a GEMM epilogue every vector
    // instruction is exposed, and the result is rounded to bf16 or compared at 1e-4
    const float sig = __builtin_amdgcn_rcpf(1.0f + __expf(-gate));
    const float silu = gate * sig;
    dgate = (dh * up) * (silu + sig * (1.0f - silu));
    dup = dh * silu;
}

// What the staged epilogue of gemm_store_tile reads back from memory (the old C or the residual it adds to; gate and up of
// the SwiGLU-backward epilogue), requested when the kernel starts instead of band by band behind the epilogue's fences,
// where every pass of every band waits a memory latency of its own with nothing else running on the CU.  One 16-byte
// packet per band, pass and tensor: bf16 C only.  SECOND: the kernel also holds the `up` packets (the instantiations for
// the SwiGLU backward).  Every member is written on every path, so the packets stay in registers.
template <int BM, int BN, int WGM, int WGN, bool SECOND>
struct TileEpilogueReads {
    static constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, LPR = WN / 8, PASSES = 32 * LPR / 64;
    static constexpr bool kSecond = SECOND;
    Pack<bf16_t> first[TM][PASSES];
    Pack<bf16_t> second[SECOND ? TM : 1][SECOND ? PASSES : 1];
    bool have_first, have_second;
    __device__ __forceinline__ void fetch(const GemmArgs& g, const bf16_t* Rsrc, bool add_old, int bz, int part, int m0, int n0, int wm, int wn, int lane) {
        const bool gate = g.gate != nullptr && SECOND;
        // partial sums of a split contraction read nothing; unaligned C takes the scalar epilogue
        const bool need = part == 0 && g.vec_c && (gate || (add_old && g.gate == nullptr));
        have_first = need;
        have_second = need && gate;
        Pack<bf16_t> zero;
#pragma unroll
        for (int e = 0; e < 8; e++) zero.set(e, 0.f);
        second[0][0] = zero;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int ps = 0; ps < PASSES; ps++) {
                const int idx = ps * 64 + lane, r = idx / LPR, cg = idx % LPR;
                const int m = m0 + wm * WM + i * 32 + r, n = n0 + wn * WN + cg * 8;
                Pack<bf16_t> v1 = zero, v2 = zero;
                if (need) {
                    if (gate) {
                        const long long at = (long long)bz * g.sC + (long long)m * g.ldc + n;
                        v1 = load_pack(static_cast<const bf16_t*>(g.gate) + at);
                        v2 = load_pack(static_cast<const bf16_t*>(g.up) + at);
                    } else {
                        v1 = load_pack(Rsrc + (long long)m * g.ldc + n);
                    }
                }
                first[i][ps] = v1;
                if constexpr (SECOND) second[i][ps] = v2;
            }
    }
};
struct NoEpilogueReads {
    static constexpr bool kSecond = false;
};

// Epilogue shared by the MFMA kernels.  Accumulator register v of lane l holds
// C[8*(v/4) + 4*(l/32) + v%4][l%32] of its 32x32 tile.  `lds_f32` is the operand LDS (LDS_BYTES bytes), idle by now
// and used as a staging area.
template <int BM, int BN, int WGM, int WGN, bool EDGE, size_t LDS_BYTES, typename TC, typename PRE = NoEpilogueReads>
__device__ __forceinline__ void gemm_store_tile(const GemmArgs& g, f32x16 (&acc)[BM / WGM / 32][BN / WGN / 32], float* lds_f32, TC* C,
                                                const TC* Rsrc, bool add_old, int bz, int split, int part, int m0, int n0, int wave,
                                                int wm, int wn, int lane, const PRE& pre = PRE{}) {
    constexpr bool kPre = !std::is_same<PRE, NoEpilogueReads>::value;  // pre.first / pre.second may hold what the staged epilogue reads
    constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 32, TN = WN / 32;
    float* P = part > 0 ? g.partial + ((long long)bz * (split - 1) + (part - 1)) * g.M * g.N : nullptr;
    constexpr int SP = WN + 4;  // staging pitch in floats
    constexpr bool kCanStage = LDS_BYTES >= (size_t)WGM * WGN * 32 * SP * sizeof(float);
    if (kCanStage && !EDGE && g.vec_c) {
        // Each wave turns its accumulators, one 32-row band at a time, through a private piece of the
        // (now idle) operand LDS so that a lane ends up with 8 consecutive columns of one row: C leaves in
        // 16-byte stores covering whole 128/256-byte row segments instead of 2- or 4-byte ones.
        float* stage = lds_f32 + wave * (32 * SP);
        constexpr int LPR = WN / 8, PASSES = 32 * LPR / 64;  // lanes per row, passes per band
        static_assert(32 * LPR % 64 == 0, "band must split evenly over the wave");
        const int c = lane & 31, gh = lane >> 5;
        const bool rotate = sizeof(TC) == 2 && g.rope && bz < g.rope_members;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            // rotary epilogue: the band's cos / sin values are requested before the accumulators go through the LDS, so that they
            // arrive while the band is staged (four pairs = 32 bytes per lane and pass)
            float4 cs[PASSES][2];
            if constexpr (sizeof(TC) == 2) {
                if (rotate) {
#pragma unroll
                    for (int ps = 0; ps < PASSES; ps++) {
                        const int idx = ps * 64 + lane, r = idx / LPR, cg = idx % LPR;
                        const int m = m0 + wm * WM + i * 32 + r, n = n0 + wn * WN + cg * 8;
                        const float4* src = reinterpret_cast<const float4*>(g.rope + (long long)(m % g.rope_seq) * (g.rope_head_dim >> 1) +
                                                                            ((n % g.rope_head_dim) >> 1));
                        cs[ps][0] = src[0];
                        cs[ps][1] = src[1];
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) stage[(8 * (v / 4) + 4 * gh + (v % 4)) * SP + j * 32 + c] = acc[i][j][v];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int ps = 0; ps < PASSES; ps++) {
                const int idx = ps * 64 + lane, r = idx / LPR, cg = idx % LPR;
                const float4 lo = *reinterpret_cast<const float4*>(stage + r * SP + cg * 8);
                const float4 hi = *reinterpret_cast<const float4*>(stage + r * SP + cg * 8 + 4);
                float val[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                const int m = m0 + wm * WM + i * 32 + r, n = n0 + wn * WN + cg * 8;
                if (P) {
                    float* dst = P + (long long)m * g.N + n;
                    *reinterpret_cast<float4*>(dst) = lo;
                    *reinterpret_cast<float4*>(dst + 4) = hi;
                } else if (g.gate) {
                    const long long at = (long long)bz * g.sC + (long long)m * g.ldc + n;
                    const TC* gsrc = static_cast<const TC*>(g.gate) + at;
                    const TC* usrc = static_cast<const TC*>(g.up) + at;
                    Pack<TC> og[8 / Pack<TC>::N], ou[8 / Pack<TC>::N];
                    bool loaded = false;
                    if constexpr (kPre && PRE::kSecond && sizeof(TC) == 2) {
                        if (pre.have_second) {
                            og[0] = pre.first[i][ps];
                            ou[0] = pre.second[i][ps];
                            loaded = true;
                        }
                    }
                    if (!loaded) {
#pragma unroll
                        for (int k = 0; k < 8 / Pack<TC>::N; k++) {
                            og[k] = load_pack(gsrc + k * Pack<TC>::N);
                            ou[k] = load_pack(usrc + k * Pack<TC>::N);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        float dgate, dup;
                        swiglu_backward_elem(og[e / Pack<TC>::N].get(e % Pack<TC>::N), ou[e / Pack<TC>::N].get(e % Pack<TC>::N), val[e], dgate, dup);
                        og[e / Pack<TC>::N].set(e % Pack<TC>::N, dgate);
                        ou[e / Pack<TC>::N].set(e % Pack<TC>::N, dup);
                    }
                    TC* d1 = C + (long long)m * g.ldc + n;
                    TC* d2 = static_cast<TC*>(g.C2) + at;
#pragma unroll
                    for (int k = 0; k < 8 / Pack<TC>::N; k++) {
                        store_pack(d1 + k * Pack<TC>::N, og[k]);
                        store_pack(d2 + k * Pack<TC>::N, ou[k]);
                    }
                } else {
                    TC* dst = C + (long long)m * g.ldc + n;
                    Pack<TC> o[8 / Pack<TC>::N];
                    if constexpr (sizeof(TC) == 2) {
                        if (rotate) {
                            // the product rounded to bf16 and then rotated, as the separate rotary kernel would find it
#pragma unroll
                            for (int q = 0; q < 2; q++) {
                                const float4 t = cs[ps][q];
                                const float a0 = to_f32(from_f32<TC>(val[4 * q])), b0 = to_f32(from_f32<TC>(val[4 * q + 1]));
                                const float a1 = to_f32(from_f32<TC>(val[4 * q + 2])), b1 = to_f32(from_f32<TC>(val[4 * q + 3]));
                                rope_rotate_forward(a0, b0, make_float2(t.x, t.y), val[4 * q], val[4 * q + 1]);
                                rope_rotate_forward(a1, b1, make_float2(t.z, t.w), val[4 * q + 2], val[4 * q + 3]);
                            }
                        }
                    }
                    if (add_old) {
                        bool loaded = false;
                        if constexpr (kPre && sizeof(TC) == 2) {
                            if (pre.have_first) {  // (never set together with a gate: that epilogue is the branch above)
                                o[0] = pre.first[i][ps];
                                loaded = true;
                            }
                        }
                        if (!loaded) {
                            const TC* src = Rsrc + (long long)m * g.ldc + n;
#pragma unroll
                            for (int k = 0; k < 8 / Pack<TC>::N; k++) o[k] = load_pack(src + k * Pack<TC>::N);
                        }
#pragma unroll
                        for (int e = 0; e < 8; e++) val[e] += o[e / Pack<TC>::N].get(e % Pack<TC>::N);
                    }
#pragma unroll
                    for (int e = 0; e < 8; e++) o[e / Pack<TC>::N].set(e % Pack<TC>::N, val[e]);
#pragma unroll
                    for (int k = 0; k < 8 / Pack<TC>::N; k++) store_pack(dst + k * Pack<TC>::N, o[k]);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + wn * WN + j * 32 + (lane & 31);
            if (EDGE && n >= g.N) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (!EDGE || m < g.M) {
                    const float val = acc[i][j][v];
                    if (P) {
                        P[(long long)m * g.N + n] = val;
                    } else if (g.gate) {
                        const long long at = (long long)bz * g.sC + (long long)m * g.ldc + n;
                        float dgate, dup;
                        swiglu_backward_elem(to_f32(static_cast<const TC*>(g.gate)[at]), to_f32(static_cast<const TC*>(g.up)[at]), val, dgate, dup);
                        C[(long long)m * g.ldc + n] = from_f32<TC>(dgate);
                        static_cast<TC*>(g.C2)[at] = from_f32<TC>(dup);
                    } else {
                        TC* dst = C + (long long)m * g.ldc + n;
                        *dst = from_f32<TC>(add_old ? to_f32(Rsrc[(long long)m * g.ldc + n]) + val : val);
                    }
                }
            }
        }
}

// ---- MFMA kernel with operands loaded straight into LDS ------------------------------------------
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory into LDS without passing through
// registers: no staging registers, no LDS store instructions, no address arithmetic per chunk.  One wave
// instruction fills 1 KB of consecutive LDS, so the tiles are unpadded and their rows are chunk-permuted
// (lds_swz in device_utils.cuh) to keep the operand reads free of bank conflicts.
// Three LDS stages: slab kt is multiplied while slabs kt+1 and kt+2 are in flight, one barrier per slab.
// The loads are issued from inline assembly so that waiting for them stays in this file's hands
// (vmcnt counts them in issue order); the kernel has no other vector memory loads in its main loop.
template <int ROWS, bool KC, int BK, int WAVES>
struct DirectOperandTile {
    static constexpr int LDS_ROW = KC ? BK : ROWS;  // elements of one LDS row = one contiguous run of the operand in memory
    static constexpr int ELEMS = ROWS * BK;
    static constexpr int CPR = LDS_ROW / 8;         // 16-byte chunks per LDS row
    static constexpr int RPB = 64 / CPR;            // LDS rows filled by one wave instruction
    static constexpr int LOADS = ELEMS / 512 / WAVES;  // wave instructions per wave and slab
    static_assert(CPR >= 4 && 64 % CPR == 0 && ELEMS % (512 * WAVES) == 0, "slab must split into whole 1 KB wave loads");

    // LDS row and (permuted) chunk this lane fetches in load i of its wave
    static __device__ __forceinline__ void lane_chunk(int i, int wave, int lane, int& row, int& chunk) {
        row = (wave * LOADS + i) * RPB + lane / CPR;
        chunk = (lane % CPR) ^ lds_swz<LDS_ROW * 2>(row);
    }
    static __device__ __forceinline__ int lds_block(int i, int wave) { return (wave * LOADS + i) * 512; }  // element offset in the tile

    // MFMA operand of the 32 operand rows starting at `row0` for contraction offsets ks..ks+15 (same register
    // contents as OperandTile::fragment)
    static __device__ __forceinline__ bf16x8 fragment(const bf16_t* tile, int row0, int ks, int lane) {
        if (KC) {
            const int r = row0 + (lane & 31);
            return *reinterpret_cast<const bf16x8*>(tile + r * BK + ((((ks >> 3) + (lane >> 5)) ^ lds_swz<BK * 2>(r)) << 3));
        }
        const int L = lane & 15, half = (lane >> 4) & 1;
        const int k = ks + 8 * (lane >> 5) + (L >> 2), col = row0 + 16 * half + 4 * (L & 3);
        const bf16_t* p_lo = tile + k * ROWS + ((((col >> 3) ^ lds_swz<ROWS * 2>(k)) << 3) | (col & 7));
        const bf16_t* p_hi = tile + (k + 4) * ROWS + ((((col >> 3) ^ lds_swz<ROWS * 2>(k + 4)) << 3) | (col & 7));
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p_lo));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p_hi));
        bf16x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    }
};

typedef __attribute__((address_space(3))) void* lds_void_ptr;
// one wave instruction: lane l's 16 bytes at `src` land at lds_dst + 16*l (lds_dst is wave-uniform)
__device__ __forceinline__ void load_to_lds_16(const void* src, bf16_t* lds_dst) {
    const unsigned lds_addr = (unsigned)(size_t)(lds_void_ptr)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "m0");
}
// the same with a wave-uniform 64-bit base and a 32-bit byte offset per lane (below 2 GiB): the base is two scalar
// registers and the offset does not change from slab to slab, so a load costs no vector arithmetic
__device__ __forceinline__ void load_to_lds_16(const void* base, unsigned lane_offset, bf16_t* lds_dst) {
    const unsigned lds_addr = (unsigned)(size_t)(lds_void_ptr)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(lane_offset), "s"(base) : "m0");
}
template <int N>
__device__ __forceinline__ void wait_loads_but() {  // until at most N of this wave's vector memory loads are outstanding
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// barrier without the memory fence of __syncthreads (which would wait for every outstanding load)
__device__ __forceinline__ void barrier_no_fence() {
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

}  // namespace
