// GEMM family: C[M,N] (+)= op(A) * op(B), row-major, optional batch.
//
//   forward  Y  = X * W          (A [M,K], B [K,N])            Graph::matmul, src/graph/ops/linear.rs:254-262
//   dX       dA = dC * B^T       (A [M,K'], B stored [N',K'])   src/graph/ops/linear.rs:269-277
//   dW       dB = A^T * dC       (A stored [K',M'], B [K',N'])  src/graph/ops/linear.rs:279-287
//   tied lm_head / bmm with trans_b                             src/graph/ops/linear.rs:456-481, :1430-1446
//
// bf16 path: MFMA v_mfma_f32_32x32x16_bf16, f32 accumulate.  A workgroup of 4 or 8 waves owns a
// BM x BN tile of C; each wave owns a 64x64 part of it made of 32x32 MFMA tiles.  K is walked in slabs of
// 64 (32 for odd K) through LDS, one barrier per slab, with the following slabs' global loads in flight during
// the current slab's MFMAs.  Two kernels here: gemm_mfma_direct_kernel loads its operands straight into three LDS
// stages (whole-tile shapes, 256x128 tile); gemm_mfma_kernel stages them through registers into two LDS
// buffers and handles edges.  A third one, gemm_wide.hip (256x256 tiles of four 128x128 wave tiles), takes the weight
// gradients with enough tiles.  The MFMA operand registers want 8 consecutive k per lane: a k-contiguous
// operand gets them with one ds_read_b128, an operand stored the other way round with two
// ds_read_b64_tr_b16 (LDS transpose reads), so dX, dW and the forward GEMM all stream their operands through
// LDS as plain 16-byte copies.
//
// f32 path and odd shapes: a plain LDS-tiled FMA kernel (64x64 tile, 4x4 per thread).
#include "gemm_common.cuh"

namespace {

// ---- MFMA kernel -------------------------------------------------------------------------
// A_KC: A is stored [M][K] (k contiguous); otherwise [K][M].  B_KC: B is stored [N][K];
// otherwise [K][N].  Either way a slab travels global -> registers -> LDS as straight 16-byte
// copies in its memory order:
//   k-contiguous operand : LDS tile [rows][BK + 8];  MFMA operand = one ds_read_b128
//   other order          : LDS tile [BK][rows + 16]; MFMA operand = two ds_read_b64_tr_b16, the
//                          LDS transpose read that hands a lane 4 consecutive k of one column
// so no operand is ever transposed element by element.
template <int ROWS, bool KC, int BK, int THREADS>
struct OperandTile {
    static constexpr int PITCH = KC ? BK + 8 : ROWS + 32;  // ROWS + 32: the transpose reads of a half-wave hit 64 distinct banks
    static constexpr int ELEMS = KC ? ROWS * PITCH : BK * PITCH;
    static constexpr int CHUNKS = ROWS * BK / 8 / THREADS;
    static_assert(CHUNKS >= 1 && CHUNKS * THREADS * 8 == ROWS * BK, "slab must split evenly over the threads");  // 16-byte chunks per thread per slab

    // global coordinates (row = m or n, k) of chunk `c` of thread `tid`
    static __device__ __forceinline__ void chunk_coords(int c, int tid, int& row, int& k) {
        const int chunk = c * THREADS + tid;
        if (KC) {
            row = chunk / (BK / 8);
            k = (chunk % (BK / 8)) * 8;
        } else {
            k = chunk / (ROWS / 8);
            row = (chunk % (ROWS / 8)) * 8;
        }
    }
    template <bool EDGE>
    static __device__ __forceinline__ bf16x8 load(const bf16_t* base, int ld, int row0, int k0, int row_limit, int k_limit, int c, int tid) {
        int row, k;
        chunk_coords(c, tid, row, k);
        row += row0;
        k += k0;
        const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if (EDGE && (row >= row_limit || k >= k_limit)) return zero8;
        return *reinterpret_cast<const bf16x8*>(KC ? base + (long long)row * ld + k : base + (long long)k * ld + row);
    }
    static __device__ __forceinline__ void store(bf16_t* tile, bf16x8 v, int c, int tid) {
        int row, k;
        chunk_coords(c, tid, row, k);
        *reinterpret_cast<bf16x8*>(KC ? tile + row * PITCH + k : tile + k * PITCH + row) = v;
    }
    // MFMA operand of the 32 rows starting at `row0` for contraction offsets ks..ks+15:
    // lane l holds row row0 + l%32 and k = ks + 8*(l/32) + 0..7.
    static __device__ __forceinline__ bf16x8 fragment(const bf16_t* tile, int row0, int ks, int lane) {
        if (KC) return *reinterpret_cast<const bf16x8*>(tile + (row0 + (lane & 31)) * PITCH + ks + 8 * (lane >> 5));
        const int L = lane & 15, half = (lane >> 4) & 1;
        const bf16_t* p = tile + (ks + 8 * (lane >> 5) + (L >> 2)) * PITCH + row0 + 16 * half + 4 * (L & 3);
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr)(p + 4 * PITCH));
        bf16x8 r;
        r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
        r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
        return r;
    }
};

// WGM x WGN waves share a BM x BN tile of C.  EDGE = false is for shapes that are whole multiples
// of the tile in M, N and K: no bounds checks anywhere.
template <int BM, int BN, int BK, int WGM, int WGN, bool A_KC, bool B_KC, bool EDGE, typename TC>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_kernel(GemmArgs g) {
    constexpr int THREADS = 64 * WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;      // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wave
    using TA = OperandTile<BM, A_KC, BK, THREADS>;
    using TB = OperandTile<BN, B_KC, BK, THREADS>;
    __shared__ __attribute__((aligned(16))) bf16_t lds[2][TA::ELEMS + TB::ELEMS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int split = g.split > 1 ? g.split : 1;
    const int bz = blockIdx.z / split, part = blockIdx.z % split;
    const int k_lo = part * g.k_part, k_hi = split > 1 ? min(g.K, k_lo + g.k_part) : g.K;
    const bf16_t* A = static_cast<const bf16_t*>(g.A) + (long long)bz * g.sA;
    const bf16_t* B = static_cast<const bf16_t*>(g.B) + (long long)bz * g.sB;
    TC* C = static_cast<TC*>(g.C) + (long long)bz * g.sC;
    // what the epilogue adds to the product: the old C (accumulate), a residual tensor, or nothing
    const TC* Rsrc = g.R ? static_cast<const TC*>(g.R) + (long long)bz * g.sC : C;
    const bool add_old = g.accumulate || g.R != nullptr;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // Slab hand-over.  While slab kt is multiplied out of one LDS buffer, slab kt+1 sits in registers
    // (its global loads were issued a whole slab earlier).  After the MFMAs of each contraction step a
    // share of those registers is stored into the other LDS buffer and immediately refilled with
    // slab kt+2, so LDS writes and global loads are spread between the MFMAs instead of piling up in
    // front of the barrier.  Slabs past the end are clamped to the last one: they are loaded and
    // stored like any other and never read.
    constexpr int KSTEPS = BK / 16, NCH = TA::CHUNKS + TB::CHUNKS;
    bf16x8 r[NCH];
    auto load_chunk = [&](int h, int slab) {
        // the slab's segment (uniform): selected with scalar selects, no branch in the main loop
        int k0 = k_lo + slab * BK, lda = g.lda, ldb = g.ldb;
        const bf16_t* Ap = A;
        const bf16_t* Bp = B;
        if (g.nseg > 1) {
            const bool s1 = k0 >= g.seg_end[0], s2 = g.nseg > 2 && k0 >= g.seg_end[1];
            Ap = s2 ? static_cast<const bf16_t*>(g.A_seg[1]) : s1 ? static_cast<const bf16_t*>(g.A_seg[0]) : A;
            Bp = s2 ? static_cast<const bf16_t*>(g.B_seg[1]) : s1 ? static_cast<const bf16_t*>(g.B_seg[0]) : B;
            lda = s2 ? g.lda_seg[1] : s1 ? g.lda_seg[0] : lda;
            ldb = s2 ? g.ldb_seg[1] : s1 ? g.ldb_seg[0] : ldb;
            k0 -= s2 ? g.seg_end[1] : s1 ? g.seg_end[0] : 0;
        }
        if (h < TA::CHUNKS) r[h] = TA::template load<EDGE>(Ap, lda, m0, k0, g.M, k_hi, h, tid);
        else r[h] = TB::template load<EDGE>(Bp, ldb, n0, k0, g.N, k_hi, h - TA::CHUNKS, tid);
    };
    auto store_chunk = [&](int h, int buf) {
        if (h < TA::CHUNKS) TA::store(lds[buf], r[h], h, tid);
        else TB::store(lds[buf] + TA::ELEMS, r[h], h - TA::CHUNKS, tid);
    };
    constexpr int kReads = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);  // LDS read instructions per step

    const int nk = (k_hi - k_lo + BK - 1) / BK;
#pragma unroll
    for (int h = 0; h < NCH; h++) load_chunk(h, 0);
#pragma unroll
    for (int h = 0; h < NCH; h++) store_chunk(h, 0);
#pragma unroll
    for (int h = 0; h < NCH; h++) load_chunk(h, min(1, nk - 1));
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        const bf16_t* As = lds[buf];
        const bf16_t* Bs = lds[buf] + TA::ELEMS;
        const int refill = min(kt + 2, nk - 1);
        static_for<KSTEPS>([&](auto st_c) {
            constexpr int st = decltype(st_c)::value;
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = TA::fragment(As, wm * WM + i * 32, st * 16, lane);
#pragma unroll
            for (int j = 0; j < TN; j++) b[j] = TB::fragment(Bs, wn * WN + j * 32, st * 16, lane);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            constexpr int h_lo = st * NCH / KSTEPS, h_hi = (st + 1) * NCH / KSTEPS;  // this step's share of the hand-over
#pragma unroll
            for (int h = h_lo; h < h_hi; h++) {
                store_chunk(h, buf ^ 1);
                load_chunk(h, refill);
            }
            if (!EDGE) {  // pin the order: operand reads, then MFMA / LDS write / global load in turn
                __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
#pragma unroll
                for (int h = h_lo; h < h_hi; h++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (h_hi - h_lo), 0);
            }
        });
        __syncthreads();
    }

    gemm_store_tile<BM, BN, WGM, WGN, EDGE, sizeof(lds), TC>(g, acc, reinterpret_cast<float*>(&lds[0][0]), C, Rsrc, add_old, bz, split, part,
                                                             m0, n0, wave, wm, wn, lane);
}

// For shapes that are whole multiples of the tile in M, N and K (no bounds checks anywhere).
// PIPE: the operand registers of contraction step st+1 are read between the MFMAs of step st.
// SWIGLU_BWD: an instantiation of its own for the launches with the SwiGLU-backward epilogue (the epilogue itself is
// chosen by g.gate in every instantiation), so that a kernel trace lists them apart from the plain products: they run
// beside a weight-gradient GEMM on the side stream, which stretches their durations.
template <int BM, int BN, int BK, int WGM, int WGN, bool A_KC, bool B_KC, typename TC, bool PIPE, bool SWIGLU_BWD = false>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_direct_kernel(GemmArgs g) {
    if (SWIGLU_BWD && !g.gate) return;
    constexpr int WAVES = WGM * WGN, STAGES = 3;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int KSTEPS = BK / 16;
    using TA = DirectOperandTile<BM, A_KC, BK, WAVES>;
    using TB = DirectOperandTile<BN, B_KC, BK, WAVES>;
    constexpr int NLOADS = TA::LOADS + TB::LOADS;
    __shared__ __attribute__((aligned(1024))) bf16_t lds[STAGES][TA::ELEMS + TB::ELEMS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    // Tile order: the workgroups resident at one time (about one per CU, in dispatch order) should cover a
    // compact block of C, so that the A and B panels they stream fit the caches together: C is walked in groups
    // of g.tile_group N tiles, all M tiles of a group before the next group, N index fastest inside a group.
    int mt = blockIdx.y, nt = blockIdx.x, zz = blockIdx.z, gt = blockIdx.x;
    if (g.split > 1) {
        // Parts of a split contraction: the tiles of one part read the same K range of A and B, and nothing else does.  In
        // dispatch order (x fastest, z = part slowest, handed to the XCDs round-robin) every XCD would hold tiles of every
        // part and fetch every K range into its own L2; renumbered, an XCD holds whole parts.
        const int gx = gridDim.x, gy = gridDim.y;
        const int lin = xcd_contiguous_id(blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z), gx * gy * gridDim.z);
        nt = gt = lin % gx;
        mt = (lin / gx) % gy;
        zz = lin / (gx * gy);
    } else if (g.tile_group < 0) {
        xcd_block_tile<4, 8>(blockIdx.y * gridDim.x + blockIdx.x, gridDim.y, gridDim.x, mt, nt);
    } else if (g.tile_group > 0) {
        const int m_tiles = gridDim.y, n_tiles = gridDim.x;
        const int lin = blockIdx.y * n_tiles + blockIdx.x, per_group = g.tile_group * m_tiles;
        const int grp = lin / per_group, within = lin % per_group;
        const int width = min(g.tile_group, n_tiles - grp * g.tile_group);
        mt = within / width;
        nt = grp * g.tile_group + within % width;
    }
    if (g.ngroup > 0) {  // which product this tile belongs to (uniform); static indices keep the tables in scalar registers
        const int t = gt;
        int first = 0;
        long long partial_off = g.grp_partial_off[0];
        g.A = g.grp_A[0]; g.B = g.grp_B[0]; g.C = g.grp_C[0]; g.N = g.grp_N[0];
#pragma unroll
        for (int q = 1; q < kMaxGroup; q++)
            if (q < g.ngroup && t >= g.grp_tile_end[q - 1]) {
                first = g.grp_tile_end[q - 1];
                partial_off = g.grp_partial_off[q];
                g.A = g.grp_A[q]; g.B = g.grp_B[q]; g.C = g.grp_C[q]; g.N = g.grp_N[q];
            }
        if (g.split > 1) g.partial += partial_off;
        const int n_tiles = g.N / BN;
        mt = (t - first) / n_tiles;
        nt = (t - first) % n_tiles;
        g.ldc = g.N;
        if (!B_KC) g.ldb = g.N;
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int split = g.split > 1 ? g.split : 1;
    const int bz = zz / split, part = zz % split;
    const int k_lo = part * g.k_part, k_hi = split > 1 ? min(g.K, k_lo + g.k_part) : g.K;
    const bf16_t* A = static_cast<const bf16_t*>(g.A) + (long long)bz * g.sA;
    const bf16_t* B = static_cast<const bf16_t*>(g.B) + (long long)bz * g.sB;
    TC* C = static_cast<TC*>(g.C) + (long long)bz * g.sC;
    const TC* Rsrc = g.R ? static_cast<const TC*>(g.R) + (long long)bz * g.sC : C;
    const bool add_old = g.accumulate || g.R != nullptr;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // this lane's chunk of each of its wave's loads (the same for every slab), as a byte offset from the slab's origin for
    // the leading dimensions in force; a segment of the contraction with other leading dimensions recomputes them
    int a_row[TA::LOADS], a_chunk[TA::LOADS], b_row[TB::LOADS], b_chunk[TB::LOADS];
    unsigned a_off[TA::LOADS], b_off[TB::LOADS];
#pragma unroll
    for (int i = 0; i < TA::LOADS; i++) TA::lane_chunk(i, wave, lane, a_row[i], a_chunk[i]);
#pragma unroll
    for (int i = 0; i < TB::LOADS; i++) TB::lane_chunk(i, wave, lane, b_row[i], b_chunk[i]);
    int off_lda = -1, off_ldb = -1;
    auto set_offsets = [&](int lda, int ldb) {
        if (lda != off_lda) {
#pragma unroll
            for (int i = 0; i < TA::LOADS; i++) a_off[i] = (unsigned)(a_row[i] * lda + a_chunk[i] * 8) * 2u;
            off_lda = lda;
        }
        if (ldb != off_ldb) {
#pragma unroll
            for (int i = 0; i < TB::LOADS; i++) b_off[i] = (unsigned)(b_row[i] * ldb + b_chunk[i] * 8) * 2u;
            off_ldb = ldb;
        }
    };

    // Where a slab's loads come from and go to (uniform values): the slab's K segment is picked with scalar selects.
    struct SlabSource {
        const bf16_t *a0, *b0;
        int lda, ldb;
        bf16_t *As, *Bs;
    };
    auto locate = [&](int slab, int stage) {
        int k0 = k_lo + slab * BK, lda = g.lda, ldb = g.ldb;
        const bf16_t* Ap = A;
        const bf16_t* Bp = B;
        if (g.nseg > 1) {
            const bool s1 = k0 >= g.seg_end[0], s2 = g.nseg > 2 && k0 >= g.seg_end[1];
            Ap = s2 ? static_cast<const bf16_t*>(g.A_seg[1]) : s1 ? static_cast<const bf16_t*>(g.A_seg[0]) : A;
            Bp = s2 ? static_cast<const bf16_t*>(g.B_seg[1]) : s1 ? static_cast<const bf16_t*>(g.B_seg[0]) : B;
            lda = s2 ? g.lda_seg[1] : s1 ? g.lda_seg[0] : lda;
            ldb = s2 ? g.ldb_seg[1] : s1 ? g.ldb_seg[0] : ldb;
            k0 -= s2 ? g.seg_end[1] : s1 ? g.seg_end[0] : 0;
        }
        SlabSource src;
        // slab origin: an LDS row is an operand row (k-contiguous storage) or a contraction index (the other storage)
        src.a0 = A_KC ? Ap + (long long)m0 * lda + k0 : Ap + (long long)k0 * lda + m0;
        src.b0 = B_KC ? Bp + (long long)n0 * ldb + k0 : Bp + (long long)k0 * ldb + n0;
        src.lda = lda;
        src.ldb = ldb;
        set_offsets(lda, ldb);  // (uniform; changes only where a segment with other leading dimensions begins)
        src.As = lds[stage];
        src.Bs = lds[stage] + TA::ELEMS;
        return src;
    };
    // loads h_lo..h_hi-1 of the NLOADS this wave issues per slab
    auto issue = [&](const SlabSource& src, auto h_lo_c, auto h_hi_c) {
        constexpr int h_lo = decltype(h_lo_c)::value, h_hi = decltype(h_hi_c)::value;
#pragma unroll
        for (int h = h_lo; h < h_hi; h++) {
            if (h < TA::LOADS) load_to_lds_16(src.a0, a_off[h], src.As + TA::lds_block(h, wave));
            else load_to_lds_16(src.b0, b_off[h - TA::LOADS], src.Bs + TB::lds_block(h - TA::LOADS, wave));
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using IN = std::integral_constant<int, NLOADS>;
    const int nk = (k_hi - k_lo) / BK;
    // One workgroup per CU (slabs of 64) and bf16 C: what the epilogue adds to or multiplies with travels with the first slabs.
    constexpr bool kPrefetch = sizeof(TC) == 2 && BK == 64;
    using Pre = std::conditional_t<kPrefetch, TileEpilogueReads<BM, BN, WGM, WGN, SWIGLU_BWD>, NoEpilogueReads>;
    Pre pre;
    if constexpr (kPrefetch) pre.fetch(g, reinterpret_cast<const bf16_t*>(Rsrc), add_old, bz, part, m0, n0, wm, wn, lane);
    issue(locate(0, 0), I0{}, IN{});
    if (nk > 1) issue(locate(1, 1), I0{}, IN{});
    int stage = 0;
    // One slab.  REFILL: the loads of slab kt+2 are issued, spread over the contraction steps behind each step's
    // MFMAs, into the stage that held slab kt-1.  The last two slabs run the body without them.
    auto slab = [&](int kt, auto refill_c) {
        constexpr bool REFILL = decltype(refill_c)::value;
        // slab kt has landed when at most the loads of slab kt+1 are outstanding
        if (REFILL || kt + 1 < nk) wait_loads_but<NLOADS>();
        else wait_loads_but<0>();
        barrier_no_fence();  // slab kt is complete in LDS; every wave is done with slab kt-1
        __builtin_amdgcn_s_setprio(2);  // a wave multiplying a slab goes ahead of one still waiting for its loads (worth ~0.3 % of the step)
        const SlabSource next = locate(REFILL ? kt + 2 : kt, stage == 0 ? 2 : stage - 1);
        const bf16_t* As = lds[stage];
        const bf16_t* Bs = lds[stage] + TA::ELEMS;
        if (PIPE) {
            // operand registers of step st+1 are read from LDS while the MFMAs of step st run
            bf16x8 a[2][TM], b[2][TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[0][i] = TA::fragment(As, wm * WM + i * 32, 0, lane);
#pragma unroll
            for (int j = 0; j < TN; j++) b[0][j] = TB::fragment(Bs, wn * WN + j * 32, 0, lane);
            constexpr int kReadsStep = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);
            __builtin_amdgcn_sched_group_barrier(0x100, kReadsStep, 0);  // step 0's reads, so that the read groups below are the next step's
            static_for<KSTEPS>([&](auto st_c) {
                constexpr int st = decltype(st_c)::value;
                if (st + 1 < KSTEPS) {
#pragma unroll
                    for (int i = 0; i < TM; i++) a[(st + 1) & 1][i] = TA::fragment(As, wm * WM + i * 32, (st + 1) * 16, lane);
#pragma unroll
                    for (int j = 0; j < TN; j++) b[(st + 1) & 1][j] = TB::fragment(Bs, wn * WN + j * 32, (st + 1) * 16, lane);
                }
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[st & 1][i], b[st & 1][j], acc[i][j], 0, 0, 0);
                if (REFILL)
                    issue(next, std::integral_constant<int, st * NLOADS / KSTEPS>{}, std::integral_constant<int, (st + 1) * NLOADS / KSTEPS>{});
                // pin the order: each MFMA of this step is followed by its share of the next step's operand reads
                if (st + 1 < KSTEPS) {
                    static_for<TM * TN>([&](auto m_c) {
                        constexpr int mi = decltype(m_c)::value;
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        constexpr int r_lo = mi * kReadsStep / (TM * TN), r_hi = (mi + 1) * kReadsStep / (TM * TN);
                        if (r_hi > r_lo) __builtin_amdgcn_sched_group_barrier(0x100, r_hi - r_lo, 0);
                    });
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
                }
            });
        } else
        static_for<KSTEPS>([&](auto st_c) {
            constexpr int st = decltype(st_c)::value;
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = TA::fragment(As, wm * WM + i * 32, st * 16, lane);
#pragma unroll
            for (int j = 0; j < TN; j++) b[j] = TB::fragment(Bs, wn * WN + j * 32, st * 16, lane);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            if (REFILL)
                issue(next, std::integral_constant<int, st * NLOADS / KSTEPS>{}, std::integral_constant<int, (st + 1) * NLOADS / KSTEPS>{});
        });
        __builtin_amdgcn_s_setprio(0);
        stage = stage == 2 ? 0 : stage + 1;
    };
    int kt = 0;
    for (; kt + 2 < nk; kt++) slab(kt, std::true_type{});
    for (; kt < nk; kt++) slab(kt, std::false_type{});
    barrier_no_fence();  // the staging epilogue reuses the operand LDS
    gemm_store_tile<BM, BN, WGM, WGN, false, sizeof(lds), TC, Pre>(g, acc, reinterpret_cast<float*>(&lds[0][0]), C, Rsrc, add_old, bz, split, part,
                                                                   m0, n0, wave, wm, wn, lane, pre);
}

// ---- gate and up projections with the SwiGLU in the epilogue ----------------------------------------
// G = X Wg, U = X Wu, H = silu(G) * U (src/nn/transformer.rs:41-46) as one kernel: a workgroup multiplies its 256 rows of
// X against the same 128 columns of both weights, so every A operand register feeds twice as many MFMAs (a 64 x 128
// wave tile in effect: a sixth fewer LDS reads per MFMA than two separate products), and H is formed from the f32
// accumulators.  Same machinery as gemm_mfma_direct_kernel: direct-to-LDS loads, three stages, slabs of 32.
struct SwigluForwardArgs {
    const bf16_t* X;   // [M, K]
    const bf16_t* Wg;  // [K, N]
    const bf16_t* Wu;  // [K, N]
    bf16_t* G;         // [M, N]
    bf16_t* U;
    bf16_t* H;
    int M, N, K;
    int tile_group;    // PLAIN: N tiles per group of the tile order (see gemm_mfma_direct_kernel), 0 = row-major
};
// PLAIN: no SwiGLU; the same main loop as one 256 x 256 tile of C = X W (Wg = W, Wu = W + 128 columns, G = C, U = C + 128
// columns, N = row length of W and C; blockIdx.x enumerates the (M / 256) * (N / 256) tiles).
template <bool PLAIN>
__global__ __launch_bounds__(512) void gemm_swiglu_forward_kernel(SwigluForwardArgs g) {
    constexpr int BM = 256, BN = 128, BK = 32, WGN = 2, WAVES = 8, STAGES = 3;
    constexpr int WM = 64, WN = 64, TM = 2, TN = 2, KSTEPS = BK / 16;
    using TA = DirectOperandTile<BM, true, BK, WAVES>;
    using TB = DirectOperandTile<BN, false, BK, WAVES>;
    constexpr int NLOADS = TA::LOADS + 2 * TB::LOADS, STAGE_ELEMS = TA::ELEMS + 2 * TB::ELEMS;
    __shared__ __attribute__((aligned(1024))) bf16_t lds[STAGES][STAGE_ELEMS];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    int mt = blockIdx.y, nt = blockIdx.x;
    if (PLAIN) {
        const int n_tiles = g.N / (2 * BN), m_tiles = g.M / BM, lin = blockIdx.x;
        mt = lin / n_tiles;
        nt = lin % n_tiles;
        if (g.tile_group > 0) {
            const int per_group = g.tile_group * m_tiles, grp = lin / per_group, within = lin % per_group;
            const int width = min(g.tile_group, n_tiles - grp * g.tile_group);
            mt = within / width;
            nt = grp * g.tile_group + within % width;
        }
    }
    const int m0 = mt * BM, n0 = nt * (PLAIN ? 2 * BN : BN);

    f32x16 accg[TM][TN], accu[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) { accg[i][j][v] = 0.f; accu[i][j][v] = 0.f; }

    // this lane's chunk of each of its wave's loads, as a byte offset from the slab's origin (the same for every slab: a load
    // takes the slab's origin in scalar registers and this offset, no vector arithmetic)
    unsigned a_off[TA::LOADS], b_off[TB::LOADS];
#pragma unroll
    for (int i = 0; i < TA::LOADS; i++) {
        int row, chunk;
        TA::lane_chunk(i, wave, lane, row, chunk);
        a_off[i] = (unsigned)(row * g.K + chunk * 8) * 2u;
    }
#pragma unroll
    for (int i = 0; i < TB::LOADS; i++) {
        int row, chunk;
        TB::lane_chunk(i, wave, lane, row, chunk);
        b_off[i] = (unsigned)(row * g.N + chunk * 8) * 2u;
    }
    // loads h_lo..h_hi-1 of the NLOADS this wave issues per slab: X rows, then the Wg and Wu slabs
    auto issue = [&](int slab, int stage, auto h_lo_c, auto h_hi_c) {
        constexpr int h_lo = decltype(h_lo_c)::value, h_hi = decltype(h_hi_c)::value;
        const int k0 = slab * BK;
        bf16_t* st = lds[stage];
        const bf16_t* x0 = g.X + (long long)m0 * g.K + k0;
        const long long w_origin = (long long)k0 * g.N + n0;
#pragma unroll
        for (int h = h_lo; h < h_hi; h++) {
            if (h < TA::LOADS) {
                load_to_lds_16(x0, a_off[h], st + TA::lds_block(h, wave));
            } else {
                const int hb = (h - TA::LOADS) % TB::LOADS;
                const bool second = h - TA::LOADS >= TB::LOADS;
                const bf16_t* W = second ? g.Wu : g.Wg;
                load_to_lds_16(W + w_origin, b_off[hb], st + TA::ELEMS + (second ? TB::ELEMS : 0) + TB::lds_block(hb, wave));
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using IN = std::integral_constant<int, NLOADS>;
    const int nk = g.K / BK;
    issue(0, 0, I0{}, IN{});
    if (nk > 1) issue(1, 1, I0{}, IN{});
    int stage = 0;
    auto slab = [&](int kt, auto refill_c) {
        constexpr bool REFILL = decltype(refill_c)::value;
        if (REFILL || kt + 1 < nk) wait_loads_but<NLOADS>();
        else wait_loads_but<0>();
        barrier_no_fence();
        __builtin_amdgcn_s_setprio(2);
        const int refill_stage = stage == 0 ? 2 : stage - 1;
        const bf16_t* As = lds[stage];
        const bf16_t* Bg = lds[stage] + TA::ELEMS;
        const bf16_t* Bu = Bg + TB::ELEMS;
        static_for<KSTEPS>([&](auto st_c) {
            constexpr int st = decltype(st_c)::value;
            bf16x8 a[TM], bg[TN], bu[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = TA::fragment(As, wm * WM + i * 32, st * 16, lane);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                bg[j] = TB::fragment(Bg, wn * WN + j * 32, st * 16, lane);
                bu[j] = TB::fragment(Bu, wn * WN + j * 32, st * 16, lane);
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    accg[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], bg[j], accg[i][j], 0, 0, 0);
                    accu[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], bu[j], accu[i][j], 0, 0, 0);
                }
            if (REFILL) issue(kt + 2, refill_stage, std::integral_constant<int, st * NLOADS / KSTEPS>{}, std::integral_constant<int, (st + 1) * NLOADS / KSTEPS>{});
        });
        __builtin_amdgcn_s_setprio(0);
        stage = stage == 2 ? 0 : stage + 1;
    };
    int kt = 0;
    for (; kt + 2 < nk; kt++) slab(kt, std::true_type{});
    for (; kt < nk; kt++) slab(kt, std::false_type{});
    barrier_no_fence();  // the staging epilogue reuses the operand LDS

    // Epilogue: as in gemm_store_tile, each wave turns a 32-row band of its accumulators through its private LDS
    // area so that a lane ends up with 8 consecutive columns of one row; here twice (G, then U) before H is formed.
    constexpr int SP = WN + 4, LPR = WN / 8, PASSES = 32 * LPR / 64;
    static_assert(sizeof(lds) >= (size_t)WAVES * 32 * SP * sizeof(float), "staging area does not fit the operand LDS");
    float* stage_f = reinterpret_cast<float*>(&lds[0][0]) + wave * (32 * SP);
    const int c = lane & 31, gh = lane >> 5;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        float vg[PASSES][8], vu[PASSES][8];
#pragma unroll
        for (int which = 0; which < 2; which++) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    stage_f[(8 * (v / 4) + 4 * gh + (v % 4)) * SP + j * 32 + c] = which == 0 ? accg[i][j][v] : accu[i][j][v];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int ps = 0; ps < PASSES; ps++) {
                const int idx = ps * 64 + lane, r = idx / LPR, cg = idx % LPR;
                const float4 lo = *reinterpret_cast<const float4*>(stage_f + r * SP + cg * 8);
                const float4 hi = *reinterpret_cast<const float4*>(stage_f + r * SP + cg * 8 + 4);
                float* dst = which == 0 ? vg[ps] : vu[ps];
                dst[0] = lo.x; dst[1] = lo.y; dst[2] = lo.z; dst[3] = lo.w;
                dst[4] = hi.x; dst[5] = hi.y; dst[6] = hi.z; dst[7] = hi.w;
            }
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ps++) {
            const int idx = ps * 64 + lane, r = idx / LPR, cg = idx % LPR;
            const long long at = (long long)(m0 + wm * WM + i * 32 + r) * g.N + n0 + wn * WN + cg * 8;
            bf16x8 og, ou, oh;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                // the outputs the backward pass reads are the rounded ones, so H is formed from them as the separate kernel would
                og[e] = (bf16_t)vg[ps][e];
                ou[e] = (bf16_t)vu[ps][e];
                if (!PLAIN) {
                    const float gv = (float)og[e], uv = (float)ou[e];
                    oh[e] = (bf16_t)(gv * __builtin_amdgcn_rcpf(1.0f + __expf(-gv)) * uv);  // 1-ulp reciprocal: the result is rounded to bf16
                }
            }
            *reinterpret_cast<bf16x8*>(g.G + at) = og;
            *reinterpret_cast<bf16x8*>(g.U + at) = ou;
            if (!PLAIN) *reinterpret_cast<bf16x8*>(g.H + at) = oh;
        }
    }
}

// C += partial[0] + partial[1] + ... in that order, one thread per 4 consecutive elements of a row.
template <typename TC>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmArgs g, int batch) {
    const long long per = (long long)g.M * g.N, quads = per / 4;
    const long long q = (long long)blockIdx.x * 256 + threadIdx.x;
    if (q >= quads * batch) return;
    const long long bz = q / quads, e = (q % quads) * 4;
    const int m = (int)(e / g.N), n = (int)(e % g.N);
    TC* dst = static_cast<TC*>(g.C) + bz * g.sC + (long long)m * g.ldc + n;
    float sum[4];
#pragma unroll
    for (int i = 0; i < 4; i++) sum[i] = to_f32(dst[i]);  // part 0 already went into C (assigned or accumulated)
    // the partials are fetched eight at a time (independent loads in flight) and added in part order
    const float* part0 = g.partial + bz * (g.split - 1) * per + e;
    for (int p0 = 0; p0 < g.split - 1; p0 += 8) {
        float4 x[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            x[i] = p0 + i < g.split - 1 ? *reinterpret_cast<const float4*>(part0 + (long long)(p0 + i) * per) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (p0 + i < g.split - 1) {
                sum[0] += x[i].x; sum[1] += x[i].y; sum[2] += x[i].z; sum[3] += x[i].w;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) dst[i] = from_f32<TC>(sum[i]);
}

// The same for a grouped launch: blockIdx.y is the product (f32 results, no batch).
__global__ __launch_bounds__(256) void gemm_splitk_reduce_grouped_kernel(GemmArgs g) {
    const int p = blockIdx.y;
    const int N = g.grp_N[p];
    const long long per = (long long)g.M * N, quads = per / 4;
    const long long q = (long long)blockIdx.x * 256 + threadIdx.x;
    if (q >= quads) return;
    float* dst = static_cast<float*>(g.grp_C[p]) + q * 4;
    float4 sum = *reinterpret_cast<const float4*>(dst);  // part 0 already went into C (assigned or accumulated)
    const float* part0 = g.partial + g.grp_partial_off[p] + q * 4;
    for (int p0 = 0; p0 < g.split - 1; p0 += 8) {
        float4 x[8];
#pragma unroll
        for (int i = 0; i < 8; i++)
            x[i] = p0 + i < g.split - 1 ? *reinterpret_cast<const float4*>(part0 + (long long)(p0 + i) * per) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (p0 + i < g.split - 1) {
                sum.x += x[i].x; sum.y += x[i].y; sum.z += x[i].z; sum.w += x[i].w;
            }
        }
    }
    *reinterpret_cast<float4*>(dst) = sum;
}

// ---- generic kernel (f32, or bf16 with shapes the MFMA kernel does not take) ---------------
template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs g, int trans_a, int trans_b) {
    constexpr int T = 64, KT = 16;
    __shared__ float As[KT][T + 1], Bs[KT][T + 1];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
    const TA* A = static_cast<const TA*>(g.A) + (long long)blockIdx.z * g.sA;
    const TA* B = static_cast<const TA*>(g.B) + (long long)blockIdx.z * g.sB;
    TC* C = static_cast<TC*>(g.C) + (long long)blockIdx.z * g.sC;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < g.K; k0 += KT) {
        for (int e = tid; e < T * KT; e += 256) {
            // read along the operand's contiguous dimension
            int kk, mm;
            if (trans_a) { kk = e / T; mm = e % T; } else { mm = e / KT; kk = e % KT; }
            const int m = m0 + mm, k = k0 + kk;
            float v = 0.f;
            if (m < g.M && k < g.K) v = to_f32(trans_a ? A[(long long)k * g.lda + m] : A[(long long)m * g.lda + k]);
            As[kk][mm] = v;
            int kb, nn;
            if (trans_b) { nn = e / KT; kb = e % KT; } else { kb = e / T; nn = e % T; }
            const int n = n0 + nn, k2 = k0 + kb;
            float w = 0.f;
            if (n < g.N && k2 < g.K) w = to_f32(trans_b ? B[(long long)n * g.ldb + k2] : B[(long long)k2 * g.ldb + n]);
            Bs[kb][nn] = w;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KT; kk++) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < g.M && n < g.N) {
                TC* dst = C + (long long)m * g.ldc + n;
                const TC* src = g.R ? static_cast<const TC*>(g.R) + (long long)blockIdx.z * g.sC + (long long)m * g.ldc + n : dst;
                *dst = from_f32<TC>((g.accumulate || g.R) ? to_f32(*src) + acc[i][j] : acc[i][j]);
            }
        }
}

template <int BM, int BN, int BK, int WGM, int WGN, bool EDGE, typename TC>
void launch_mfma_t(eisen_ctx* ctx, const GemmArgs& g, bool a_kc, bool b_kc, int batch) {
    dim3 grid((unsigned)eisen_ceil_div(g.N, BN), (unsigned)eisen_ceil_div(g.M, BM), (unsigned)(batch * (g.split > 1 ? g.split : 1)));
    constexpr int T = 64 * WGM * WGN;
    if (a_kc && b_kc) gemm_mfma_kernel<BM, BN, BK, WGM, WGN, true, true, EDGE, TC><<<grid, T, 0, ctx->stream>>>(g);
    else if (a_kc && !b_kc) gemm_mfma_kernel<BM, BN, BK, WGM, WGN, true, false, EDGE, TC><<<grid, T, 0, ctx->stream>>>(g);
    else if (!a_kc && b_kc) gemm_mfma_kernel<BM, BN, BK, WGM, WGN, false, true, EDGE, TC><<<grid, T, 0, ctx->stream>>>(g);
    else gemm_mfma_kernel<BM, BN, BK, WGM, WGN, false, false, EDGE, TC><<<grid, T, 0, ctx->stream>>>(g);
}
template <int BM, int BN, int BK, int WGM, int WGN>
void launch_mfma_direct(eisen_ctx* ctx, GemmArgs g, bool a_kc, bool b_kc, int batch, int dtype_c) {
    // grids many N tiles wide walk C in groups of 32 N tiles (measured on the 32000-column lm_head GEMMs: 4 % and
    // 10 % faster than row-major order); narrower grids are a few rounds of workgroups anyway
    g.tile_group = g.N / BN >= 64 ? 32 : 0;
    // 256-row tiles of narrower grids: blocks of 4 x 8 tiles per XCD (tile_group < 0, see xcd_block_tile; 1-5 % faster on the
    // products of a 4096-token step with contractions of 2048 to 32000)
    if (g.tile_group == 0 && g.ngroup == 0 && BM == 256) g.tile_group = -1;
    // reading step st+1's operand registers between step st's MFMAs gains 2-4 % except in the slab-32 kernels of the
    // dW shapes (two steps per slab, two or three workgroups per CU already overlapping), where it loses
    const bool pipe = a_kc || b_kc || BK == 64;
    dim3 grid((unsigned)(g.N / BN), (unsigned)(g.M / BM), (unsigned)(batch * (g.split > 1 ? g.split : 1)));
    constexpr int T = 64 * WGM * WGN;
#define EISEN_DIRECT(AK, BKC, TC) do { if (pipe) gemm_mfma_direct_kernel<BM, BN, BK, WGM, WGN, AK, BKC, TC, true><<<grid, T, 0, ctx->stream>>>(g); else gemm_mfma_direct_kernel<BM, BN, BK, WGM, WGN, AK, BKC, TC, false><<<grid, T, 0, ctx->stream>>>(g); } while (0)
    if (dtype_c == EISEN_BF16) {
        if (a_kc && b_kc) EISEN_DIRECT(true, true, bf16_t);
        else if (a_kc) EISEN_DIRECT(true, false, bf16_t);
        else if (b_kc) EISEN_DIRECT(false, true, bf16_t);
        else EISEN_DIRECT(false, false, bf16_t);
    } else {
        if (a_kc && b_kc) EISEN_DIRECT(true, true, float);
        else if (a_kc) EISEN_DIRECT(true, false, float);
        else if (b_kc) EISEN_DIRECT(false, true, float);
        else EISEN_DIRECT(false, false, float);
    }
#undef EISEN_DIRECT
}
template <int BM, int BN, int BK, int WGM, int WGN>
void launch_mfma_c(eisen_ctx* ctx, const GemmArgs& g, bool a_kc, bool b_kc, int batch, int dtype_c) {
    const bool edge = g.M % BM != 0 || g.N % BN != 0 || g.K % BK != 0 || (g.split > 1 && g.k_part % BK != 0);
    if (dtype_c == EISEN_BF16) {
        if (edge) launch_mfma_t<BM, BN, BK, WGM, WGN, true, bf16_t>(ctx, g, a_kc, b_kc, batch);
        else launch_mfma_t<BM, BN, BK, WGM, WGN, false, bf16_t>(ctx, g, a_kc, b_kc, batch);
    } else {
        if (edge) launch_mfma_t<BM, BN, BK, WGM, WGN, true, float>(ctx, g, a_kc, b_kc, batch);
        else launch_mfma_t<BM, BN, BK, WGM, WGN, false, float>(ctx, g, a_kc, b_kc, batch);
    }
}

template <typename TA, typename TC>
void launch_generic(eisen_ctx* ctx, const GemmArgs& g, int trans_a, int trans_b, int batch) {
    dim3 grid((unsigned)eisen_ceil_div(g.N, 64), (unsigned)eisen_ceil_div(g.M, 64), (unsigned)batch);
    gemm_generic_kernel<TA, TC><<<grid, 256, 0, ctx->stream>>>(g, trans_a, trans_b);
}

}  // namespace

// Internal entry shared by eisen_hip_gemm and eisen_hip_bmm.
struct KSegments {  // further (A, B, K) segments after the first one
    int n = 0;
    const void* A[2];
    const void* B[2];
    size_t K[2];
};
struct SwigluBackwardEpilogue {  // see GemmArgs::gate
    const void* gate;
    const void* up;
    void* dup;
};
struct RopeEpilogue {  // see GemmArgs::rope
    size_t members, seq, head_dim;
};
constexpr int kEpilogueNotFusable = -7001;  // internal: the shape takes a kernel without the fused epilogue
static int gemm_common(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                       int trans_b, size_t M, size_t N, size_t K, size_t batch, long long sA, long long sB, long long sC,
                       int accumulate, const char* who, const KSegments* segs = nullptr, const void* residual = nullptr,
                       const SwigluBackwardEpilogue* swiglu = nullptr, const RopeEpilogue* rope = nullptr) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, A && B && C, EISEN_E_ARG, "%s: null pointer", who);
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype_ab) && eisen_dtype_ok(dtype_c), EISEN_E_ARG, "%s: unknown dtype", who);
    EISEN_REQUIRE(ctx, !(dtype_ab == EISEN_F32 && dtype_c == EISEN_BF16), EISEN_E_ARG, "%s: f32 operands with bf16 output is not a supported combination", who);
    EISEN_REQUIRE(ctx, M < (size_t(1) << 30) && N < (size_t(1) << 30) && K < (size_t(1) << 30) && batch < 65536, EISEN_E_SHAPE, "%s: dimension out of range", who);
    if (M == 0 || N == 0 || batch == 0) return 0;
    const int n_more = segs ? segs->n : 0;
    if (n_more > 0) {
        // one launch needs bf16 operands, no batch and every segment a whole number of 64-deep slabs;
        // anything else runs as one accumulating GEMM per segment
        bool one = dtype_ab == EISEN_BF16 && batch == 1 && K % 64 == 0 && K > 0 && n_more <= 2 && eisen_aligned(A, 16) && eisen_aligned(B, 16) &&
                   (trans_a ? M % 8 == 0 : true) && (trans_b ? true : N % 8 == 0);
        for (int i = 0; i < n_more && one; i++)
            one = segs->A[i] && segs->B[i] && segs->K[i] % 64 == 0 && segs->K[i] > 0 && eisen_aligned(segs->A[i], 16) && eisen_aligned(segs->B[i], 16);
        if (!one) {
            int rc = gemm_common(ctx, A, B, C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, batch, sA, sB, sC, accumulate, who);
            for (int i = 0; i < n_more && !rc; i++)
                rc = gemm_common(ctx, segs->A[i], segs->B[i], C, dtype_ab, dtype_c, trans_a, trans_b, M, N, segs->K[i], batch, sA, sB, sC, 1, who);
            return rc;
        }
    }
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.lda = (int)(trans_a ? M : K);
    g.ldb = (int)(trans_b ? K : N);
    g.ldc = (int)N;
    g.sA = sA; g.sB = sB; g.sC = sC;
    g.accumulate = accumulate;
    g.R = residual;
    g.vec_c = (!residual || eisen_aligned(residual, 16)) && eisen_aligned(C, 16) && N % 8 == 0 && (sC * eisen_dtype_size(dtype_c)) % 16 == 0;
    if (n_more > 0) {
        size_t end = K;
        for (int i = 0; i < n_more; i++) {
            g.A_seg[i] = segs->A[i];
            g.B_seg[i] = segs->B[i];
            g.lda_seg[i] = (int)(trans_a ? M : segs->K[i]);
            g.ldb_seg[i] = (int)(trans_b ? segs->K[i] : N);
            g.seg_end[i] = (int)end;   // segment i+1 starts where the previous ones end
            end += segs->K[i];
        }
        g.nseg = n_more + 1;
        K = end;                       // from here on: the whole contraction
        g.K = (int)K;
        EISEN_REQUIRE(ctx, K < (size_t(1) << 30), EISEN_E_SHAPE, "%s: dimension out of range", who);
    }
    if (K == 0) {  // empty contraction: C (+)= 0
        if (!accumulate) {
            for (size_t b = 0; b < batch; b++) {
                int rc = eisen_hip_memset_zero(ctx, (char*)C + b * sC * eisen_dtype_size(dtype_c), M * N * eisen_dtype_size(dtype_c));
                if (rc) return rc;
            }
        }
        return 0;
    }
    const bool a_kc = !trans_a, b_kc = trans_b != 0;
    bool mfma_ok = dtype_ab == EISEN_BF16 && eisen_aligned(A, 16) && eisen_aligned(B, 16) && g.lda % 8 == 0 && g.ldb % 8 == 0 &&
                   sA % 8 == 0 && sB % 8 == 0;
    // the contiguous dimension of each operand must be a whole number of 8-element chunks
    if (a_kc) mfma_ok = mfma_ok && K % 8 == 0; else mfma_ok = mfma_ok && M % 8 == 0;
    if (b_kc) mfma_ok = mfma_ok && K % 8 == 0; else mfma_ok = mfma_ok && N % 8 == 0;
    EISEN_REQUIRE(ctx, n_more == 0 || mfma_ok, EISEN_E_ARG, "%s: segmented contraction reached a shape the MFMA kernel does not take", who);
    if (swiglu) {
        if (!mfma_ok) return kEpilogueNotFusable;
        g.gate = swiglu->gate;
        g.up = swiglu->up;
        g.C2 = swiglu->dup;
        g.vec_c = g.vec_c && eisen_aligned(swiglu->gate, 16) && eisen_aligned(swiglu->up, 16) && eisen_aligned(swiglu->dup, 16);
    }
    // profile key = one kernel instantiation (operand orders, types, tile), so the event timing
    // lines up with a profiler's per-kernel rows
    char pname[64];
    const long long tiles128 = (long long)eisen_ceil_div(M, 128) * eisen_ceil_div(N, 128) * batch;
    const bool big_tile = tiles128 >= 256 || (M >= 128 && N >= 128 && tiles128 >= 128);
    // Few output tiles and a long contraction (the dW of a narrow projection): cut K so that every CU
    // gets a tile.  Part 0 writes C as usual, the other parts go to an f32 scratch that a second kernel
    // adds to C in a fixed order, so the result does not depend on scheduling.
    int split = 1;
    if (mfma_ok && N % 4 == 0 && K >= 1024 && n_more == 0 && !swiglu) {
        const bool t128 = M >= 128 && N >= 128;
        const long long tiles = t128 ? tiles128 : (long long)eisen_ceil_div(M, 64) * eisen_ceil_div(N, 64) * batch;
        const size_t slab = t128 ? 64 : 32, min_part = t128 ? 512 : 256;
        // (a bf16 result pays for a second kernel that rounds the sum: measured worth it from parts of 2048 up, M = 8192, N = 256:
        //  K = 1024 17.1 us whole against 23.4 us in two parts, K = 2048 25.4 against 26.4, K = 8192 76.0 against 56.9)
        if (tiles <= 128 && (dtype_c != EISEN_BF16 || K >= 4096))
            while (split < 32 && tiles * split * 2 <= 256 && K / (split * 2) >= min_part && K % (split * 2 * slab) == 0) split *= 2;
    }
    const bool split128 = split > 1 && M >= 128 && N >= 128;
    // the direct-to-LDS kernels address a slab by a scalar base and a 32-bit byte offset per lane (up to 256 rows of a leading dimension)
    bool ld_small = g.lda < (1 << 22) && g.ldb < (1 << 22);
    for (int i = 0; i + 1 < g.nseg; i++) ld_small = ld_small && g.lda_seg[i] < (1 << 22) && g.ldb_seg[i] < (1 << 22);
    // 256x128 tiles only when they fill whole rounds of the 256 CUs well (one workgroup per CU)
    const long long wide_tiles = (long long)(M / 256) * (N / 128) * batch;
    const bool wide = mfma_ok && ld_small && split == 1 && big_tile && M % 256 == 0 && N % 128 == 0 && K % 64 == 0 && wide_tiles >= 256 &&
                      (double)wide_tiles / (double)(256 * ((wide_tiles + 255) / 256)) >= 0.85;
    const bool wide32 = mfma_ok && ld_small && split == 1 && n_more == 0 && !a_kc && !b_kc && M % 256 == 0 && N % 128 == 0 && K % 64 == 0 &&
                        (wide_tiles >= 512 || (wide_tiles >= 300 && !wide));
    // 256 x 256 tiles (the gate/up kernel's main loop: an A operand register feeds twice the MFMAs) where the grid still
    // has three rounds of them: the lm_head forward (1035 against 980 TFLOP/s at 4096 x 32000 x 2048)
    if (rope) {
        // the rotation lives in the staged epilogue of the whole-tile kernels; any other shape is the caller's to rotate
        // (256x128x64 and 128x128x64 direct-to-LDS kernels, the 64x64x32 kernel without bounds checks: all three stage C through
        // the LDS, where gemm_store_tile rotates)
        const bool whole128 = big_tile && M % 128 == 0 && N % 128 == 0 && K % 64 == 0;
        const bool whole64 = !big_tile && M % 64 == 0 && N % 64 == 0 && K % 32 == 0;
        static_assert(2 * (OperandTile<64, true, 32, 256>::ELEMS + OperandTile<64, false, 32, 256>::ELEMS) * sizeof(bf16_t) >= 4 * 32 * (32 + 4) * sizeof(float),
                      "the 64x64x32 kernel's LDS must hold its staged C bands");
        const bool fits = mfma_ok && split == 1 && n_more == 0 && dtype_c == EISEN_BF16 && !residual && !swiglu && !accumulate && g.vec_c && a_kc && !b_kc &&
                          (wide || whole128 || whole64) && rope->head_dim % 8 == 0 && N % rope->head_dim == 0 && rope->seq > 0 && rope->seq < (size_t(1) << 24) &&
                          rope->head_dim < (size_t(1) << 24);
        if (!fits) return kEpilogueNotFusable;
        int rc = eisen_rope_table_get(ctx, rope->seq, rope->head_dim, &g.rope);
        if (rc) return rc;
        g.rope_seq = (int)rope->seq;
        g.rope_head_dim = (int)rope->head_dim;
        g.rope_members = (int)std::min<size_t>(rope->members, batch);
    }
    const bool wide256 = mfma_ok && ld_small && split == 1 && n_more == 0 && a_kc && !b_kc && batch == 1 && dtype_c == EISEN_BF16 && !residual && !swiglu && !rope &&
                         !accumulate && M % 256 == 0 && N % 256 == 0 && K % 32 == 0 && (M / 256) * (N / 256) >= 768 && eisen_aligned(C, 16);
    if (wide256) {
        SwigluForwardArgs a{static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(B), static_cast<const bf16_t*>(B) + 128, static_cast<bf16_t*>(C),
                            static_cast<bf16_t*>(C) + 128,  nullptr,                        (int)M,                             (int)N, (int)K,
                            N / 256 >= 32 ? 16 : 0};
        EisenProfScope prof(ctx, "gemm_nn_bf16_bf16out_256x256x32", 2.0 * (double)M * (double)N * (double)K, true);
        gemm_swiglu_forward_kernel<true><<<dim3((unsigned)((M / 256) * (N / 256)), 1, 1), 512, 0, ctx->stream>>>(a);
        EISEN_LAUNCH_CHECK(ctx, who);
        return 0;
    }
    // 256 x 256 tiles of four 128 x 128 wave tiles (gemm_wide.hip).  Weight gradients (both operands through the slow
    // transposing LDS reads): 15-25 % ahead of the 256x128x32 kernel from 176 tiles up (the 5632 x 2048 and 2048 x 5632
    // gradients, 0.69 of a round of workgroups).
    const long long tiles256 = (long long)(M / 256) * (long long)(N / 256);
    const bool wide_tn = !a_kc && !b_kc && tiles256 >= 176;
    if (mfma_ok && split == 1 && n_more == 0 && !swiglu && wide_tn && M >= 256 && N >= 256 && eisen_gemm_wide_supports(g, a_kc, b_kc, (int)batch, dtype_c)) {
        snprintf(pname, sizeof(pname), "gemm_%s%s_bf16_%s_256x256x32", trans_a ? "t" : "n", trans_b ? "t" : "n", dtype_c == EISEN_BF16 ? "bf16out" : "f32out");
        EisenProfScope prof(ctx, pname, 2.0 * (double)M * (double)N * (double)K, true);
        g.tile_group = N / 256 >= 32 ? 16 : 0;
        eisen_gemm_launch_wide(ctx, g, a_kc, b_kc, dtype_c);
        EISEN_LAUNCH_CHECK(ctx, who);
        return 0;
    }
    const char* tile = !mfma_ok ? "fma64x64" : wide32 ? "256x128x32" : wide ? "256x128x64" : (big_tile || split128) ? (K % 64 == 0 && !(!a_kc && !b_kc && M % 128 == 0 && N % 128 == 0 && tiles128 * split >= 512) ? "128x128x64" : "128x128x32") : "64x64x32";
    snprintf(pname, sizeof(pname), "gemm_%s%s_%s_%s_%s%s", trans_a ? "t" : "n", trans_b ? "t" : "n", dtype_ab == EISEN_BF16 ? "bf16" : "f32",
             dtype_c == EISEN_BF16 ? "bf16out" : "f32out", tile, split > 1 ? "_splitk" : swiglu ? "_swiglu_bwd" : rope ? "_rope" : "");
    EisenProfScope prof(ctx, pname, 2.0 * (double)M * (double)N * (double)K * (double)batch, true);
    if (mfma_ok) {
        if (split > 1) {
            void* ws = nullptr;
            int rc = eisen_workspace(ctx, (size_t)batch * (split - 1) * M * N * sizeof(float), &ws);
            if (rc) return rc;
            g.split = split;
            g.k_part = (int)(K / split);
            g.partial = static_cast<float*>(ws);
        }
        // Tile choice (measured on MI355X at the config-5 shapes): 256x128 with 8 waves and operands loaded
        // straight into three LDS stages is the fastest kernel whenever the shape is a whole number of such tiles
        // and they fill the CUs evenly (it is 5-13 % ahead of the same tile staged through registers); other
        // large shapes run 128x128 (direct-to-LDS with 8 waves when the shape is whole tiles, else register-staged with 4).  64x64 is for problems with few tiles.
        if (wide32) {
            // both operands through the (slower) transposing LDS reads and more than one tile per CU: slabs of 32 need
            // half the LDS, so two workgroups share a CU and cover each other's barrier waits and epilogues (6-7 % faster
            // than slabs of 64; at 352 tiles, the down projection's dW, still 11 % faster than 704 tiles of 128x128x32)
            launch_mfma_direct<256, 128, 32, 4, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
        } else if (wide && swiglu && a_kc && b_kc && dtype_c == EISEN_BF16 && batch == 1) {
            g.tile_group = g.N / 128 >= 64 ? 32 : 0;
            gemm_mfma_direct_kernel<256, 128, 64, 4, 2, true, true, bf16_t, true, true><<<dim3((unsigned)(g.N / 128), (unsigned)(g.M / 256), 1), 512, 0, ctx->stream>>>(g);
        } else if (wide) {
            launch_mfma_direct<256, 128, 64, 4, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
        } else if (big_tile || split128) {
            // whole tiles: the direct-to-LDS kernel (one workgroup per CU) is up to 16 % ahead when the grid has at most
            // one tile per CU and level with the register-staged kernel (two workgroups per CU) beyond that
            const bool whole = ld_small && M % 128 == 0 && N % 128 == 0 && K % 64 == 0 && (split == 1 || g.k_part % 64 == 0);
            // both operands through the transposing LDS reads and at least two tiles per CU: slabs of 32 let three
            // workgroups share a CU (down-projection dW 20 % faster)
            if (whole && !a_kc && !b_kc && tiles128 * split >= 512) launch_mfma_direct<128, 128, 32, 2, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
            // (slabs of 64: three stages fill most of a CU's LDS, so one workgroup per CU either way; eight waves of 32 x 64 cover
            // each other's waits where four of 64 x 64 cannot: config 4 -2 % per step, config 5's K|V launch -4 %)
            else if (whole) launch_mfma_direct<128, 128, 64, 4, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
            else if (K % 64 == 0) launch_mfma_c<128, 128, 64, 2, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
            else launch_mfma_c<128, 128, 32, 2, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
        } else {
            launch_mfma_c<64, 64, 32, 2, 2>(ctx, g, a_kc, b_kc, (int)batch, dtype_c);
        }
        if (split > 1) {
            const long long quads = (long long)M * N / 4 * batch;
            const unsigned blocks = (unsigned)((quads + 255) / 256);
            if (dtype_c == EISEN_BF16) gemm_splitk_reduce_kernel<bf16_t><<<blocks, 256, 0, ctx->stream>>>(g, (int)batch);
            else gemm_splitk_reduce_kernel<float><<<blocks, 256, 0, ctx->stream>>>(g, (int)batch);
        }
    } else if (dtype_ab == EISEN_F32) {
        launch_generic<float, float>(ctx, g, trans_a, trans_b, (int)batch);
    } else if (dtype_c == EISEN_BF16) {
        launch_generic<bf16_t, bf16_t>(ctx, g, trans_a, trans_b, (int)batch);
    } else {
        launch_generic<bf16_t, float>(ctx, g, trans_a, trans_b, (int)batch);
    }
    EISEN_LAUNCH_CHECK(ctx, who);
    return 0;
}

extern "C" int eisen_hip_gemm(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                              int trans_b, size_t M, size_t N, size_t K, int accumulate) {
    return gemm_common(ctx, A, B, C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, 1, 0, 0, 0, accumulate, "eisen_hip_gemm");
}

extern "C" int eisen_hip_bmm(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                             int trans_b, size_t batch, size_t M, size_t N, size_t K, int accumulate) {
    return gemm_common(ctx, A, B, C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, batch, (long long)(M * K), (long long)(K * N),
                       (long long)(M * N), accumulate, "eisen_hip_bmm");
}

extern "C" int eisen_hip_gemm_strided_batched(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype_ab, int dtype_c, int trans_a,
                                              int trans_b, size_t batch, size_t M, size_t N, size_t K, long long stride_a,
                                              long long stride_b, long long stride_c, int accumulate) {
    return gemm_common(ctx, A, B, C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, batch, stride_a, stride_b, stride_c, accumulate,
                       "eisen_hip_gemm_strided_batched");
}

extern "C" int eisen_hip_gemm_rope(eisen_ctx* ctx, const void* A, const void* B, void* C, int dtype, size_t batch, size_t M, size_t N, size_t K,
                                   long long stride_b, long long stride_c, size_t rope_members, size_t seq, size_t head_dim) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, A && B && C, EISEN_E_ARG, "eisen_hip_gemm_rope: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_gemm_rope: unknown dtype %d", dtype);
    EISEN_REQUIRE(ctx, rope_members <= batch, EISEN_E_ARG, "eisen_hip_gemm_rope: %zu rotated members of %zu", rope_members, batch);
    EISEN_REQUIRE(ctx, seq > 0 && M % seq == 0, EISEN_E_SHAPE, "eisen_hip_gemm_rope: %zu rows are not whole sequences of %zu", M, seq);
    EISEN_REQUIRE(ctx, head_dim >= 2 && head_dim % 2 == 0 && N % head_dim == 0, EISEN_E_SHAPE,
                  "eisen_hip_gemm_rope: %zu columns must be a multiple of an even head_dim (%zu)", N, head_dim);
    if (batch == 0 || M == 0 || N == 0) return 0;
    const RopeEpilogue rope{rope_members, seq, head_dim};
    int rc = kEpilogueNotFusable;
    if (rope_members > 0 && K > 0)
        rc = gemm_common(ctx, A, B, C, dtype, dtype, 0, 0, M, N, K, batch, 0, stride_b, stride_c, 0, "eisen_hip_gemm_rope", nullptr, nullptr, nullptr, &rope);
    if (rc != kEpilogueNotFusable) return rc;
    // the product, then the rotation in place, member by member
    rc = gemm_common(ctx, A, B, C, dtype, dtype, 0, 0, M, N, K, batch, 0, stride_b, stride_c, 0, "eisen_hip_gemm_rope");
    for (size_t b = 0; b < rope_members && !rc; b++) {
        void* Cb = static_cast<char*>(C) + (long long)b * stride_c * (long long)eisen_dtype_size(dtype);
        rc = eisen_hip_rope(ctx, Cb, Cb, dtype, M / seq, seq, N, head_dim);
    }
    return rc;
}

extern "C" int eisen_hip_gemm_ksegments(eisen_ctx* ctx, size_t n_segments, const void* const* A, const void* const* B, const size_t* K,
                                        void* C, int dtype_ab, int dtype_c, int trans_a, int trans_b, size_t M, size_t N, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, A && B && K && C && n_segments >= 1 && n_segments <= 3, EISEN_E_ARG, "eisen_hip_gemm_ksegments: 1 to 3 segments, no null pointers");
    KSegments more;
    more.n = (int)n_segments - 1;
    for (int i = 0; i < more.n; i++) {
        more.A[i] = A[i + 1];
        more.B[i] = B[i + 1];
        more.K[i] = K[i + 1];
    }
    return gemm_common(ctx, A[0], B[0], C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K[0], 1, 0, 0, 0, accumulate, "eisen_hip_gemm_ksegments", &more);
}

extern "C" int eisen_hip_gemm_residual(eisen_ctx* ctx, const void* A, const void* B, const void* R, void* C, int dtype_ab, int dtype_c,
                                       int trans_a, int trans_b, size_t M, size_t N, size_t K) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, R != nullptr, EISEN_E_ARG, "eisen_hip_gemm_residual: null residual");
    if (K == 0) {  // C = R
        if (R != C && M * N > 0) return eisen_hip_dtod(ctx, C, R, M * N * eisen_dtype_size(dtype_c));
        return 0;
    }
    return gemm_common(ctx, A, B, C, dtype_ab, dtype_c, trans_a, trans_b, M, N, K, 1, 0, 0, 0, 0, "eisen_hip_gemm_residual", nullptr, R);
}

extern "C" int eisen_hip_gemm_swiglu_forward(eisen_ctx* ctx, const void* X, const void* Wg, const void* Wu, void* G, void* U, void* H, int dtype,
                                             size_t M, size_t N, size_t K) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, X && Wg && Wu && G && U && H, EISEN_E_ARG, "eisen_hip_gemm_swiglu_forward: null pointer");
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "eisen_hip_gemm_swiglu_forward: unknown dtype %d", dtype);
    if (M * N == 0) return 0;
    const bool fused = dtype == EISEN_BF16 && M % 256 == 0 && N % 128 == 0 && K % 32 == 0 && K >= 32 && (M / 256) * (N / 128) >= 256 &&
                       M / 256 <= 65535 && M < (size_t(1) << 30) && N < (size_t(1) << 22) && K < (size_t(1) << 22) && eisen_aligned(X, 16) && eisen_aligned(Wg, 16) &&
                       eisen_aligned(Wu, 16) && eisen_aligned(G, 16) && eisen_aligned(U, 16) && eisen_aligned(H, 16);
    if (fused) {
        SwigluForwardArgs a{static_cast<const bf16_t*>(X), static_cast<const bf16_t*>(Wg), static_cast<const bf16_t*>(Wu), static_cast<bf16_t*>(G),
                            static_cast<bf16_t*>(U),       static_cast<bf16_t*>(H),        (int)M,                          (int)N, (int)K, 0};
        EisenProfScope prof(ctx, "gemm_nn_bf16_swiglu_256x128x32", 4.0 * (double)M * (double)N * (double)K, true);
        gemm_swiglu_forward_kernel<false><<<dim3((unsigned)(N / 128), (unsigned)(M / 256), 1), 512, 0, ctx->stream>>>(a);
        EISEN_LAUNCH_CHECK(ctx, "eisen_hip_gemm_swiglu_forward");
        return 0;
    }
    int rc = gemm_common(ctx, X, Wg, G, dtype, dtype, 0, 0, M, N, K, 1, 0, 0, 0, 0, "eisen_hip_gemm_swiglu_forward");
    if (!rc) rc = gemm_common(ctx, X, Wu, U, dtype, dtype, 0, 0, M, N, K, 1, 0, 0, 0, 0, "eisen_hip_gemm_swiglu_forward");
    if (!rc) rc = eisen_hip_swiglu(ctx, G, U, H, dtype, M * N);
    return rc;
}

extern "C" int eisen_hip_gemm_grouped(eisen_ctx* ctx, size_t n, const void* const* A, const void* const* B, void* const* C, const size_t* N,
                                      int dtype_ab, int dtype_c, int trans_a, int trans_b, size_t M, size_t K, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, n >= 1 && n <= (size_t)kMaxGroup && A && B && C && N, EISEN_E_ARG, "eisen_hip_gemm_grouped: 1 to 8 products, no null pointers");
    // One launch when every product is a whole number of 128x128 tiles of the dW form (bf16 operands stored [K][M] and
    // [K][N], f32 result) and together they give every CU at least two tiles; otherwise one launch per product.
    // (leading dimensions below 2^22: the direct-to-LDS kernels address a slab by a scalar base and a 32-bit byte offset per lane)
    bool grouped = n >= 2 && dtype_ab == EISEN_BF16 && dtype_c == EISEN_F32 && trans_a && !trans_b && M % 128 == 0 && K % 64 == 0 && K > 0 &&
                   M < (size_t(1) << 22) && K < (size_t(1) << 30);
    long long tiles = 0;
    for (size_t p = 0; p < n && grouped; p++) {
        grouped = A[p] && B[p] && C[p] && N[p] > 0 && N[p] % 128 == 0 && N[p] < (size_t(1) << 22) && eisen_aligned(A[p], 16) && eisen_aligned(B[p], 16) &&
                  eisen_aligned(C[p], 16);
        tiles += (long long)(M / 128) * (long long)(N[p] / 128);
    }
    // 256 x 256 tiles (gemm_wide.hip) when every product is a whole number of them
    bool wide256 = grouped && M % 256 == 0;
    long long tiles256 = 0;
    for (size_t p = 0; p < n && wide256; p++) {
        wide256 = N[p] % 256 == 0;
        tiles256 += (long long)(M / 256) * (long long)(N[p] / 256);
    }
    if (wide256 && tiles256 >= 176 && tiles256 < (1ll << 30)) {
        GemmArgs g{};
        g.M = (int)M; g.K = (int)K;
        g.lda = (int)M;
        g.accumulate = accumulate;
        g.vec_c = 1;
        g.ngroup = (int)n;
        int end = 0;
        double flops = 0.0;
        for (size_t p = 0; p < n; p++) {
            g.grp_A[p] = A[p]; g.grp_B[p] = B[p]; g.grp_C[p] = C[p];
            g.grp_N[p] = (int)N[p];
            end += (int)((M / 256) * (N[p] / 256));
            g.grp_tile_end[p] = end;
            flops += 2.0 * (double)M * (double)N[p] * (double)K;
        }
        if (eisen_gemm_wide_supports(g, false, false, 1, dtype_c)) {
            EisenProfScope prof(ctx, "gemm_tn_bf16_f32out_256x256x32_grouped", flops, true);
            eisen_gemm_launch_wide(ctx, g, false, false, dtype_c);
            EISEN_LAUNCH_CHECK(ctx, "eisen_hip_gemm_grouped");
            return 0;
        }
    }
    const bool wide = grouped && M % 256 == 0 && tiles / 2 >= 300;  // 256x128x32 tiles, two workgroups per CU
    if (grouped && (wide || tiles >= 512) && tiles < (1ll << 30)) {
        const size_t bm = wide ? 256 : 128;
        GemmArgs g{};
        g.M = (int)M; g.K = (int)K;
        g.lda = (int)M;
        g.accumulate = accumulate;
        g.vec_c = 1;
        g.ngroup = (int)n;
        int end = 0;
        double flops = 0.0;
        for (size_t p = 0; p < n; p++) {
            g.grp_A[p] = A[p]; g.grp_B[p] = B[p]; g.grp_C[p] = C[p];
            g.grp_N[p] = (int)N[p];
            end += (int)((M / bm) * (N[p] / 128));
            g.grp_tile_end[p] = end;
            flops += 2.0 * (double)M * (double)N[p] * (double)K;
        }
        EisenProfScope prof(ctx, wide ? "gemm_tn_bf16_f32out_256x128x32_grouped" : "gemm_tn_bf16_f32out_128x128x32_grouped", flops, true);
        if (wide) gemm_mfma_direct_kernel<256, 128, 32, 4, 2, false, false, float, false><<<dim3((unsigned)end, 1, 1), 512, 0, ctx->stream>>>(g);
        else gemm_mfma_direct_kernel<128, 128, 32, 2, 2, false, false, float, false><<<dim3((unsigned)end, 1, 1), 256, 0, ctx->stream>>>(g);
        EISEN_LAUNCH_CHECK(ctx, "eisen_hip_gemm_grouped");
        return 0;
    }
    // Few tiles and a long contraction (the weight gradients of a narrow model: 256 x 64 ... 256 x 1024 over thousands of
    // tokens): one launch of 64 x 64 tiles over every product and every part of a split contraction, then one launch
    // that adds each product's partial results in part order.  Instead of a GEMM and a reduction per product.
    bool small = n >= 2 && dtype_ab == EISEN_BF16 && dtype_c == EISEN_F32 && trans_a && !trans_b && M % 64 == 0 && K % 32 == 0 && K >= 1024 &&
                 M < (size_t(1) << 22) && K < (size_t(1) << 30);
    long long tiles64 = 0, out_elems = 0;
    size_t max_n = 0;
    for (size_t p = 0; p < n && small; p++) {
        small = A[p] && B[p] && C[p] && N[p] > 0 && N[p] % 64 == 0 && N[p] < (size_t(1) << 22) && eisen_aligned(A[p], 16) && eisen_aligned(B[p], 16) &&
                eisen_aligned(C[p], 16);
        tiles64 += (long long)(M / 64) * (long long)(N[p] / 64);
        out_elems += (long long)M * (long long)N[p];
        max_n = std::max(max_n, N[p]);
    }
    if (small && tiles64 <= 512) {
        int split = 1;
        while (split < 32 && tiles64 * split < 1024 && K % ((size_t)split * 2 * 32) == 0 && K / ((size_t)split * 2) >= 256) split *= 2;
        if (split > 1) {
            void* ws = nullptr;
            int rc = eisen_workspace(ctx, (size_t)(split - 1) * (size_t)out_elems * sizeof(float), &ws);
            if (rc) return rc;
            GemmArgs g{};
            g.M = (int)M; g.K = (int)K;
            g.lda = (int)M;
            g.accumulate = accumulate;
            g.vec_c = 1;
            g.ngroup = (int)n;
            g.split = split;
            g.k_part = (int)(K / split);
            g.partial = static_cast<float*>(ws);
            int end = 0;
            long long off = 0;
            double flops = 0.0;
            for (size_t p = 0; p < n; p++) {
                g.grp_A[p] = A[p]; g.grp_B[p] = B[p]; g.grp_C[p] = C[p];
                g.grp_N[p] = (int)N[p];
                end += (int)((M / 64) * (N[p] / 64));
                g.grp_tile_end[p] = end;
                g.grp_partial_off[p] = off;
                off += (long long)(split - 1) * (long long)M * (long long)N[p];
                flops += 2.0 * (double)M * (double)N[p] * (double)K;
            }
            EisenProfScope prof(ctx, "gemm_tn_bf16_f32out_64x64x32_grouped_splitk", flops, true);
            gemm_mfma_direct_kernel<64, 64, 32, 1, 1, false, false, float, false><<<dim3((unsigned)end, 1, (unsigned)split), 64, 0, ctx->stream>>>(g);
            const unsigned blocks = (unsigned)eisen_ceil_div((size_t)M * max_n / 4, (size_t)256);
            gemm_splitk_reduce_grouped_kernel<<<dim3(blocks, (unsigned)n, 1), 256, 0, ctx->stream>>>(g);
            EISEN_LAUNCH_CHECK(ctx, "eisen_hip_gemm_grouped");
            return 0;
        }
    }
    for (size_t p = 0; p < n; p++) {
        const int rc = gemm_common(ctx, A[p], B[p], C[p], dtype_ab, dtype_c, trans_a, trans_b, M, N[p], K, 1, 0, 0, 0, accumulate, "eisen_hip_gemm_grouped");
        if (rc) return rc;
    }
    return 0;
}

// C_p (+)= sum_s A_ps^T B_ps: the dB += A^T dC of Graph::matmul (src/graph/ops/linear.rs:281-295) for several weights and
// several micro-batches at once.  One launch of 256 x 256 tiles whose contraction walks through the pieces when every
// shape is a whole number of tiles; otherwise one accumulating GEMM per product and piece, in piece order.
static_assert(kMaxWindowSegments == EISEN_GEMM_MAX_KSEGMENTS, "the kernel's table and the header disagree");
extern "C" int eisen_hip_gemm_grouped_ksegments(eisen_ctx* ctx, size_t n_products, size_t n_segments, const void* const* A, const void* const* B,
                                                void* const* C, const size_t* M, const size_t* N, size_t seg_k, int accumulate) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, n_products >= 1 && n_segments >= 1 && A && B && C && M && N, EISEN_E_ARG,
                  "eisen_hip_gemm_grouped_ksegments: at least one product and one piece, no null pointers");
    EISEN_REQUIRE(ctx, seg_k > 0 && seg_k < (size_t(1) << 30), EISEN_E_SHAPE, "eisen_hip_gemm_grouped_ksegments: piece length %zu out of range", seg_k);
    for (size_t p = 0; p < n_products; p++) {
        EISEN_REQUIRE(ctx, C[p] && M[p] > 0 && N[p] > 0 && M[p] < (size_t(1) << 30) && N[p] < (size_t(1) << 30), EISEN_E_ARG,
                      "eisen_hip_gemm_grouped_ksegments: product %zu has a null result or an empty shape", p);
        for (size_t s = 0; s < n_segments; s++)
            EISEN_REQUIRE(ctx, A[p * n_segments + s] && B[p * n_segments + s], EISEN_E_ARG, "eisen_hip_gemm_grouped_ksegments: product %zu piece %zu is null", p, s);
    }
    bool one = n_products < (size_t(1) << 16) && n_segments <= (size_t)kMaxWindowSegments && seg_k % 32 == 0;
    if (one) {
        std::vector<WideWindowRow> rows(n_products);
        WideWindow w{};
        w.nprod = (int)n_products;
        w.nseg = (int)n_segments;
        w.seg_slabs = (int)(seg_k / 32);
        w.accumulate = accumulate;
        long long tiles = 0;
        double flops = 0.0;
        for (size_t p = 0; p < n_products && one; p++) {
            WideWindowRow& r = rows[p];
            r.M = (int)M[p];
            r.N = (int)N[p];
            r.pad = 0;
            r.C = C[p];
            one = eisen_aligned(C[p], 16);
            for (size_t s = 0; s < (size_t)kMaxWindowSegments; s++) {
                const size_t from = p * n_segments + std::min(s, n_segments - 1);
                r.A[s] = A[from];
                r.B[s] = B[from];
                one = one && eisen_aligned(A[from], 16) && eisen_aligned(B[from], 16);
            }
            tiles += (long long)(M[p] / 256) * (long long)(N[p] / 256);
            one = one && tiles < (1ll << 30);
            r.tile_end = (int)tiles;
            flops += 2.0 * (double)M[p] * (double)N[p] * (double)seg_k * (double)n_segments;
        }
        // fewer tiles than CUs would leave most of the chip idle for the whole contraction
        one = one && tiles >= 176 && eisen_gemm_wide_window_supports(w, rows.data());
        if (one) {
            // the table, and behind it the (zeroed) counters of the meeting points: one per XCD and 32 tiles of its range
            const int meet_us = ctx->window_meet_us;
            const size_t ngrp = (size_t)((tiles / 8 + 31) / 32);
            const size_t table_bytes = rows.size() * sizeof(WideWindowRow), meet_bytes = meet_us > 0 ? 8 * ngrp * sizeof(int) : 0;
            std::vector<char> host(table_bytes + meet_bytes, 0);
            memcpy(host.data(), rows.data(), table_bytes);
            void* table = nullptr;
            int rc = eisen_hip_malloc(ctx, host.size(), &table);
            if (rc) return rc;
            rc = eisen_hip_htod(ctx, table, host.data(), host.size());
            if (!rc) {
                w.rows = static_cast<const WideWindowRow*>(table);
                if (meet_us > 0) {
                    w.meet = reinterpret_cast<int*>(static_cast<char*>(table) + table_bytes);
                    w.meet_ticks = meet_us * 100;
                }
                EisenProfScope prof(ctx, "gemm_tn_bf16_f32out_256x256x32_window", flops, true);
                eisen_gemm_launch_wide_window(ctx, w, (unsigned)tiles);
            }
            const int rc_free = eisen_hip_free(ctx, table);  // stream-ordered: reused only by later work
            if (rc) return rc;
            if (rc_free) return rc_free;
            EISEN_LAUNCH_CHECK(ctx, "eisen_hip_gemm_grouped_ksegments");
            return 0;
        }
    }
    for (size_t p = 0; p < n_products; p++)
        for (size_t s = 0; s < n_segments; s++) {
            const int rc = gemm_common(ctx, A[p * n_segments + s], B[p * n_segments + s], C[p], EISEN_BF16, EISEN_F32, 1, 0, M[p], N[p], seg_k, 1, 0, 0, 0,
                                       s == 0 ? accumulate : 1, "eisen_hip_gemm_grouped_ksegments");
            if (rc) return rc;
        }
    return 0;
}

extern "C" int eisen_hip_gemm_window_meet(eisen_ctx* ctx, int microseconds) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, microseconds >= 0 && microseconds <= 1000, EISEN_E_ARG, "eisen_hip_gemm_window_meet: %d us outside [0, 1000]", microseconds);
    ctx->window_meet_us = microseconds;
    return 0;
}

extern "C" int eisen_hip_gemm_swiglu_backward(eisen_ctx* ctx, const void* A, const void* B, const void* gate, const void* up, void* dgate,
                                              void* dup, int dtype, int trans_a, int trans_b, size_t M, size_t N, size_t K) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, gate && up && dgate && dup, EISEN_E_ARG, "eisen_hip_gemm_swiglu_backward: null pointer");
    if (M * N == 0) return 0;
    if (K > 0) {
        const SwigluBackwardEpilogue fuse{gate, up, dup};
        const int rc = gemm_common(ctx, A, B, dgate, dtype, dtype, trans_a, trans_b, M, N, K, 1, 0, 0, 0, 0, "eisen_hip_gemm_swiglu_backward", nullptr,
                                   nullptr, &fuse);
        if (rc != kEpilogueNotFusable) return rc;
    }
    // shapes and types the MFMA kernels do not take: the product through a temporary, then the element-wise kernel
    void* dh = nullptr;
    int rc = eisen_hip_malloc(ctx, M * N * eisen_dtype_size(dtype), &dh);
    if (rc) return rc;
    rc = gemm_common(ctx, A, B, dh, dtype, dtype, trans_a, trans_b, M, N, K, 1, 0, 0, 0, 0, "eisen_hip_gemm_swiglu_backward");
    if (!rc) rc = eisen_hip_swiglu_backward(ctx, gate, up, dh, dgate, dup, dtype, M * N, 0, 0);
    const int rc_free = eisen_hip_free(ctx, dh);
    return rc ? rc : rc_free;
}
