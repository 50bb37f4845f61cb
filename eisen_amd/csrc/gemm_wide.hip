// GEMM with 256 x 256 workgroup tiles made of four 128 x 128 wave tiles (bf16 operands, f32 accumulate).
//
// Every LDS read instruction of a wave costs the CU's one LDS pipe about 8 cycles whatever its width (16-byte
// reads move 128 bytes a cycle, the 8-byte transposing reads half of that), and a 32x32x16 MFMA keeps one of the
// four matrix pipes busy for 32 cycles.  A 64 x 64 wave tile reads 4 operand registers (4 to 8 LDS instructions) per
// 4 MFMAs: with eight waves the LDS pipe is as busy as the matrix pipes or busier, and the kernels of gemm.hip
// stall on it (MFMA pipes 50-58 % busy).  A 128 x 128 wave tile reads 8 operand registers per 16 MFMAs, half the
// LDS instructions per MFMA.  Its 256 accumulator registers are the whole AGPR file of a wave, so a SIMD holds one
// wave and nothing hides a stall but the wave's own instruction order: operand registers are double buffered, the
// LDS reads of contraction step s+1 and the global loads of a later slab are spread between the MFMAs of step s,
// and the one barrier per slab sits inside a run of MFMAs whose operands are already in registers.
//
// Operands travel global -> LDS with global_load_lds_dwordx4 (no staging registers) into a ring of four 32-deep
// slabs, three of them in flight; tiles are unpadded and chunk-permuted as in gemm.hip.
#include "gemm_common.cuh"

namespace {

constexpr int WBM = 256, WBN = 256, WBK = 32, WWAVES = 4, WSTAGES = 4;

// lane's 16 bytes at sbase + voff -> LDS at lds_addr + 16 * lane (lds_addr wave-uniform)
__device__ __forceinline__ void wide_load_lds_16(const void* sbase, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "m0");
}

struct NoWindow {};

// a pointer every lane holds the same value of, moved to scalar registers
template <typename T>
__device__ __forceinline__ T* uniform_pointer(T* p) {
    const unsigned long long v = reinterpret_cast<unsigned long long>(p);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return reinterpret_cast<T*>(((unsigned long long)hi << 32) | lo);
}

// WIN: the products, their shapes and the pieces of their contraction come from `w` (see WideWindow); g carries the
// flags of the epilogue only.
template <bool A_KC, bool B_KC, typename TC, bool WIN>
__global__ __launch_bounds__(256) void gemm_wide_kernel(GemmArgs g, std::conditional_t<WIN, WideWindow, NoWindow> w) {
    constexpr int TM = 4, TN = 4, WM = 128, WN = 128;
    using TA = DirectOperandTile<WBM, A_KC, WBK, WWAVES>;
    using TB = DirectOperandTile<WBN, B_KC, WBK, WWAVES>;
    constexpr int LA = TA::LOADS, LB = TB::LOADS, NLOADS = LA + LB;  // wave instructions per wave and slab
    constexpr int STAGE_ELEMS = TA::ELEMS + TB::ELEMS;
    __shared__ __attribute__((aligned(1024))) bf16_t lds[WSTAGES][STAGE_ELEMS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // which tile (and, in a grouped launch, of which product)
    int t = blockIdx.x, mt, nt;
    int prod = 0;
    if constexpr (WIN) {
        // an XCD (its own L2) works through a contiguous range of the tile order, 32 tiles at a time: with the order below
        // those are a compact block of one product's tiles, which share their operand panels in that L2
        t = xcd_contiguous_id(t, gridDim.x);
        // the first product whose tiles end after t (the table is the same for every lane: scalar loads)
        int lo = 0, hi = w.nprod - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (t >= __builtin_amdgcn_readfirstlane(w.rows[mid].tile_end)) lo = mid + 1;
            else hi = mid;
        }
        prod = lo;
        if (prod > 0) t -= __builtin_amdgcn_readfirstlane(w.rows[prod - 1].tile_end);
        const WideWindowRow& row = w.rows[prod];
        g.M = __builtin_amdgcn_readfirstlane(row.M); g.N = __builtin_amdgcn_readfirstlane(row.N);
        g.C = uniform_pointer(row.C);
        g.A = uniform_pointer(row.A[0]); g.B = uniform_pointer(row.B[0]);
        g.lda = g.M; g.ldb = g.N; g.ldc = g.N;
        g.K = w.nseg * w.seg_slabs * WBK;
    } else if (g.ngroup > 0) {
        int first = 0;
        g.A = g.grp_A[0]; g.B = g.grp_B[0]; g.C = g.grp_C[0]; g.N = g.grp_N[0];
#pragma unroll
        for (int q = 1; q < kMaxGroup; q++)
            if (q < g.ngroup && t >= g.grp_tile_end[q - 1]) {
                first = g.grp_tile_end[q - 1];
                g.A = g.grp_A[q]; g.B = g.grp_B[q]; g.C = g.grp_C[q]; g.N = g.grp_N[q];
            }
        t -= first;
        g.ldc = g.N;
        if (!B_KC) g.ldb = g.N;
    }
    if constexpr (WIN) {
        // blocks of about 32 tiles: every M tile of a few N tiles, or (a tall product of few N tiles) every N tile of a few M tiles
        const int n_tiles = g.N / WBN, m_tiles = g.M / WBM;
        const bool along_m = m_tiles > 8 && n_tiles <= 8;
        const int inner = along_m ? n_tiles : m_tiles, outer = along_m ? m_tiles : n_tiles;
        const int width_max = max(1, 32 / inner);
        const int per_group = width_max * inner, grp = t / per_group, within = t % per_group;
        const int width = min(width_max, outer - grp * width_max);
        const int in_i = within / width, out_i = grp * width_max + within % width;
        mt = along_m ? out_i : in_i;
        nt = along_m ? in_i : out_i;
    } else {
        const int n_tiles = g.N / WBN, m_tiles = g.M / WBM;
        if (g.tile_group > 0) {  // all M tiles of a group of N tiles before the next group
            const int per_group = g.tile_group * m_tiles, grp = t / per_group, within = t % per_group;
            const int width = min(g.tile_group, n_tiles - grp * g.tile_group);
            mt = within / width;
            nt = grp * g.tile_group + within % width;
        } else {
            mt = t / n_tiles;
            nt = t % n_tiles;
        }
    }
    const int m0 = mt * WBM, n0 = nt * WBN;
    if constexpr (WIN) {
        const int per = gridDim.x / 8;
        if (w.meet != nullptr && (int)blockIdx.x < per * 8) {
            if (tid == 0) {
                const int local = blockIdx.x / 8, grp = local / 32, ngrp = (per + 31) / 32;
                const int expect = min(32, per - grp * 32);
                int* c = w.meet + (blockIdx.x % 8) * ngrp + grp;
                __hip_atomic_fetch_add(c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const long long t0 = wall_clock64();
                while (__hip_atomic_load(c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < expect && wall_clock64() - t0 < w.meet_ticks)
                    __builtin_amdgcn_s_sleep(16);
            }
            __syncthreads();
        }
    }
    const bf16_t* A = static_cast<const bf16_t*>(g.A);
    const bf16_t* B = static_cast<const bf16_t*>(g.B);
    TC* C = static_cast<TC*>(g.C);
    const TC* Rsrc = g.R ? static_cast<const TC*>(g.R) : C;
    const bool add_old = g.accumulate || g.R != nullptr;

    // slab origin and per-slab advance of each operand (uniform), this lane's byte offsets inside a slab (the same
    // for every slab)
    const long long a_tile = (A_KC ? (long long)m0 * g.lda : (long long)m0) * 2;  // bytes from the operand's first element
    const long long b_tile = (B_KC ? (long long)n0 * g.ldb : (long long)n0) * 2;
    const char* a_base = reinterpret_cast<const char*>(A) + a_tile;
    const char* b_base = reinterpret_cast<const char*>(B) + b_tile;
    // WIN: where the tile's slabs start in the pieces after the first, in the order they will be needed
    const char* a_seg[kMaxWindowSegments - 1];
    const char* b_seg[kMaxWindowSegments - 1];
    int seg_left = 0;  // slabs of the current piece not yet requested
    if constexpr (WIN) {
#pragma unroll
        for (int s = 1; s < kMaxWindowSegments; s++) {
            a_seg[s - 1] = static_cast<const char*>(uniform_pointer(w.rows[prod].A[s])) + a_tile;
            b_seg[s - 1] = static_cast<const char*>(uniform_pointer(w.rows[prod].B[s])) + b_tile;
        }
        seg_left = w.seg_slabs - (WSTAGES - 1);
    }
    const long long a_step = A_KC ? (long long)WBK * 2 : (long long)WBK * g.lda * 2;
    const long long b_step = B_KC ? (long long)WBK * 2 : (long long)WBK * g.ldb * 2;
    unsigned a_off[LA], b_off[LB];
#pragma unroll
    for (int i = 0; i < LA; i++) {
        int row, chunk;
        TA::lane_chunk(i, wave, lane, row, chunk);
        a_off[i] = (unsigned)(((long long)row * g.lda + chunk * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
        int row, chunk;
        TB::lane_chunk(i, wave, lane, row, chunk);
        b_off[i] = (unsigned)(((long long)row * g.ldb + chunk * 8) * 2);
    }
    const unsigned lds0 = (unsigned)(size_t)(lds_void_ptr)(&lds[0][0]);
    // loads h_lo..h_hi-1 of the NLOADS this wave issues for the slab at (a_src, b_src) into `stage`
    auto issue = [&](const char* a_src, const char* b_src, int stage, auto h_lo_c, auto h_hi_c) {
        constexpr int h_lo = decltype(h_lo_c)::value, h_hi = decltype(h_hi_c)::value;
        const unsigned base = lds0 + stage * (STAGE_ELEMS * 2);
#pragma unroll
        for (int h = h_lo; h < h_hi; h++) {
            if (h < LA) wide_load_lds_16(a_src, a_off[h], base + TA::lds_block(h, wave) * 2);
            else wide_load_lds_16(b_src, b_off[h - LA], base + (TA::ELEMS + TB::lds_block(h - LA, wave)) * 2);
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using IN = std::integral_constant<int, NLOADS>;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const int nk = g.K / WBK;  // >= WSTAGES (checked by the launcher)
    // slabs 0 .. WSTAGES-2 go out first
    const char* a_next = a_base;
    const char* b_next = b_base;
#pragma unroll
    for (int s = 0; s < WSTAGES - 1; s++) {
        issue(a_next, b_next, s, I0{}, IN{});
        a_next += a_step;
        b_next += b_step;
    }
    bf16x8 a[2][TM], b[2][TN];
    // operand register q of a contraction step, in the order the MFMAs want them (row 0 of the wave tile first):
    // a0 b0 b1 b2 b3 a1 a2 a3
    auto read_frag = [&](auto buf_c, auto stage_c, auto ks_c, auto q_c) {
        constexpr int buf = decltype(buf_c)::value, st = decltype(stage_c)::value, ks = decltype(ks_c)::value, q = decltype(q_c)::value;
        const bf16_t* As = lds[st];
        const bf16_t* Bs = lds[st] + TA::ELEMS;
        if (q == 0) a[buf][0] = TA::fragment(As, wm * WM, ks, lane);
        else if (q <= TN) b[buf][q - 1] = TB::fragment(Bs, wn * WN + (q - 1) * 32, ks, lane);
        else a[buf][q - TN] = TA::fragment(As, wm * WM + (q - TN) * 32, ks, lane);
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C16 = std::integral_constant<int, 16>;
    wait_loads_but<(WSTAGES - 2) * NLOADS>();
    barrier_no_fence();
    static_for<TM + TN>([&](auto q_c) { read_frag(C0{}, C0{}, C0{}, q_c); });

    // One slab in stage ST: two contraction steps of 16 MFMAs, every MFMA followed by its share of the other work, in
    // exactly this order (a scheduling fence after each group).  Step 0 reads the operand registers of step 1.  Step 1
    // waits, after its first four MFMAs, for slab kt + 1 (one more slab may stay in flight), passes the barrier, then reads
    // the first operand registers of slab kt + 1 and sends the loads of slab kt + WSTAGES - 1 into the stage that slab
    // kt - 1 occupied: every wave has consumed its reads from that stage in MFMAs issued before it reached this barrier.
    // Every slab runs the same code: past the end of K the loads fetch the last slab again (into a stage nobody reads
    // any more) and the operand registers read ahead are not used.
    int to_issue = nk - (WSTAGES - 1);  // slabs not yet requested; a_next / b_next point at the next one
    auto slab = [&](auto stage_c) {
        constexpr int ST = decltype(stage_c)::value;
        constexpr int refill_stage = ST == 0 ? WSTAGES - 1 : ST - 1, next_stage = ST == WSTAGES - 1 ? 0 : ST + 1;
        using SC = std::integral_constant<int, ST>;
        using NC = std::integral_constant<int, next_stage>;
        static_for<TM * TN>([&](auto m_c) {
            constexpr int mi = decltype(m_c)::value, i = mi / TN, j = mi % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0][i], b[0][j], acc[i][j], 0, 0, 0);
            if (mi % 2 == 0) read_frag(C1{}, SC{}, C16{}, std::integral_constant<int, mi / 2>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<TN>([&](auto m_c) {
            constexpr int j = decltype(m_c)::value;
            acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1][0], b[1][j], acc[0][j], 0, 0, 0);
        });
        wait_loads_but<NLOADS>();
        barrier_no_fence();
        __builtin_amdgcn_sched_barrier(0);
        static_for<(TM - 1) * TN>([&](auto m_c) {
            constexpr int mi = decltype(m_c)::value, i = 1 + mi / TN, j = mi % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1][i], b[1][j], acc[i][j], 0, 0, 0);
            if (mi < TM + TN) read_frag(C0{}, NC{}, C0{}, std::integral_constant<int, mi < TM + TN ? mi : 0>{});
            if (mi >= (TM - 1) * TN - NLOADS)
                issue(a_next, b_next, refill_stage, std::integral_constant<int, mi - ((TM - 1) * TN - NLOADS)>{},
                      std::integral_constant<int, mi - ((TM - 1) * TN - NLOADS) + 1>{});
            __builtin_amdgcn_sched_barrier(0);
        });
        to_issue--;
        if constexpr (WIN) {
            seg_left--;
            if (to_issue > 0) {
                if (seg_left == 0) {  // the next slab is the first of the next piece
                    seg_left = w.seg_slabs;
                    a_next = a_seg[0];
                    b_next = b_seg[0];
#pragma unroll
                    for (int s = 0; s + 1 < kMaxWindowSegments - 1; s++) {
                        a_seg[s] = a_seg[s + 1];
                        b_seg[s] = b_seg[s + 1];
                    }
                } else {
                    a_next += a_step;
                    b_next += b_step;
                }
            }
        } else {
            a_next += to_issue > 0 ? a_step : 0;
            b_next += to_issue > 0 ? b_step : 0;
        }
    };
    static_assert(WSTAGES == 4, "the ring below is written out for four stages");
    for (int ring = 0; ring < nk / WSTAGES; ring++) {  // K is a whole number of rings (checked by the launcher)
        slab(std::integral_constant<int, 0>{});
        slab(std::integral_constant<int, 1>{});
        slab(std::integral_constant<int, 2>{});
        slab(std::integral_constant<int, 3>{});
    }
    wait_loads_but<0>();  // the repeated loads of the last slabs must not land in the epilogue's staging area
    barrier_no_fence();  // the staging epilogue reuses the operand LDS
    gemm_store_tile<WBM, WBN, 2, 2, false, sizeof(lds), TC>(g, acc, reinterpret_cast<float*>(&lds[0][0]), C, Rsrc, add_old, 0, 1, 0, m0, n0, wave,
                                                            wm, wn, lane);
}

}  // namespace

bool eisen_gemm_wide_supports(const GemmArgs& g, bool a_kc, bool b_kc, int batch, int dtype_c) {
    (void)dtype_c;
    if (batch != 1 || g.split > 1 || g.nseg > 1 || g.gate) return false;
    if (g.M % WBM || g.K % (WBK * WSTAGES) || g.K < WBK * WSTAGES) return false;
    if (g.ngroup > 0) {
        for (int p = 0; p < g.ngroup; p++)
            if (g.grp_N[p] % WBN) return false;
    } else if (g.N % WBN) {
        return false;
    }
    // a lane's offset inside a slab is a 32-bit number of bytes
    const long long rows_a = a_kc ? WBM : WBK, rows_b = b_kc ? WBN : WBK;
    long long ldb = g.ldb;
    if (g.ngroup > 0 && !b_kc)
        for (int p = 0; p < g.ngroup; p++) ldb = ldb > g.grp_N[p] ? ldb : g.grp_N[p];
    return rows_a * g.lda * 2 < (1ll << 31) && rows_b * ldb * 2 < (1ll << 31);
}

void eisen_gemm_launch_wide(eisen_ctx* ctx, const GemmArgs& g, bool a_kc, bool b_kc, int dtype_c) {
    unsigned tiles;
    if (g.ngroup > 0) tiles = (unsigned)g.grp_tile_end[g.ngroup - 1];
    else tiles = (unsigned)((g.M / WBM) * (g.N / WBN));
#define EISEN_WIDE(AK, BKC, TC) gemm_wide_kernel<AK, BKC, TC, false><<<dim3(tiles, 1, 1), 256, 0, ctx->stream>>>(g, NoWindow{})
    if (dtype_c == EISEN_BF16) {
        if (a_kc && b_kc) EISEN_WIDE(true, true, bf16_t);
        else if (a_kc) EISEN_WIDE(true, false, bf16_t);
        else if (b_kc) EISEN_WIDE(false, true, bf16_t);
        else EISEN_WIDE(false, false, bf16_t);
    } else {
        if (a_kc && b_kc) EISEN_WIDE(true, true, float);
        else if (a_kc) EISEN_WIDE(true, false, float);
        else if (b_kc) EISEN_WIDE(false, true, float);
        else EISEN_WIDE(false, false, float);
    }
#undef EISEN_WIDE
}

bool eisen_gemm_wide_window_supports(const WideWindow& w, const WideWindowRow* host_rows) {
    if (w.nprod < 1 || w.nseg < 1 || w.nseg > kMaxWindowSegments) return false;
    if (w.seg_slabs < WSTAGES || w.seg_slabs % WSTAGES) return false;
    if ((long long)w.nseg * w.seg_slabs * WBK >= (1ll << 31)) return false;
    for (int p = 0; p < w.nprod; p++) {
        const WideWindowRow& r = host_rows[p];
        if (r.M <= 0 || r.N <= 0 || r.M % WBM || r.N % WBN) return false;
        // a lane's offset inside a slab is a 32-bit number of bytes
        if ((long long)WBK * r.M * 2 >= (1ll << 31) || (long long)WBK * r.N * 2 >= (1ll << 31)) return false;
    }
    return true;
}

void eisen_gemm_launch_wide_window(eisen_ctx* ctx, const WideWindow& w, unsigned tiles) {
    GemmArgs g{};
    g.accumulate = w.accumulate;
    g.vec_c = 1;
    gemm_wide_kernel<false, false, float, true><<<dim3(tiles, 1, 1), 256, 0, ctx->stream>>>(g, w);
}
