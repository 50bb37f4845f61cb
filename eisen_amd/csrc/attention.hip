// Causal grouped-query flash attention, forward (saving log-sum-exp) and backward.
//
// The reference trains through the unfused chain bmm -> mul(scale) -> add(mask) -> softmax ->
// bmm with repeat_kv and three transposes around it (src/nn/attention.rs:300-375); its fused
// kernel is inference-only (src/graph/ops/attention.rs:7-18).  These kernels compute the same
// function and the same gradients without materialising [B*H, S, S] or the repeated K/V:
//   P = softmax(scale * Q K^T + causal mask),  O = P V
//   dV = P^T dO,  dP = dO V^T,  dS = P o (dP - rowsum(dO o O)),  dQ = scale dS K,  dK = scale dS^T Q
// with dK/dV summed over the query heads of a KV group (the repeat_kv backward,
// src/graph/ops/gqa.rs:168-184) inside the kernel.
//
// Tensors are addressed as base + b*stride_b + s*stride_s + h*stride_h + d, so both
// [B,S,H,hd] (what the projections produce) and [B,H,S,hd] (the reference's q_t layout) work.
//
// bf16 path (head_dim 32/64/128), v_mfma_f32_32x32x16_bf16, one wave = 32 query rows or 32 keys:
//   forward / dQ kernel: a wave keeps its Q (and dO) rows in registers as MFMA B operands and
//     walks 64-key K/V tiles staged in LDS.  Scores are produced transposed (S^T = K Q^T), so a
//     lane owns one query and the softmax statistics never leave the lane pair; P^T is already
//     in B-operand order for O^T += V^T P^T, and V^T / K^T come out of the row-major LDS tile
//     through ds_read_b64_tr_b16.
//   dK/dV kernel: a wave keeps 32 keys of K and V in registers, accumulates their dK/dV over
//     every query head of the group and every visible query tile; Q/dO tiles go through LDS.
//     No atomics anywhere: dQ has its own query-stationary pass, so results are reproducible.
// f32 path (any head_dim): one wave per query row / key row, plain FMA, for small shapes.
#include <cmath>
#include <mutex>

#include "attention_common.cuh"

namespace {

// Scratch of eisen_hip_attention_backward_noalloc: D = rowsum(dO o O) and -LSE / scale, two floats per (batch, query
// head, position).  A file-scope device array instead of a workspace allocation, so that entry point never calls an
// allocator.  Every GPU the library runs on holds its own 8 MiB copy until the process ends; the name below is only a
// host-side handle, the device address of each GPU's copy comes from hipGetSymbolAddress (eisen_attention_scratch_init).
constexpr size_t kNoAllocMaxRows = size_t(1) << 20;
static __device__ __align__(256) float g_attn_bwd_scratch[2 * kNoAllocMaxRows];
constexpr int kMaxDevices = 64;
static float* g_attn_bwd_scratch_ptr[kMaxDevices] = {nullptr};  // per device, filled once
// Every context and stream of a GPU shares that GPU's array, so calls are put in order: the event is recorded behind the
// kernels of a call and the next call's stream waits for it first (two contexts on one GPU, or the main and the side
// stream of one).  The mutex covers the two tables and the wait / launch / record sequence.
static hipEvent_t g_attn_bwd_scratch_done[kMaxDevices] = {nullptr};
static std::mutex g_attn_bwd_scratch_mu;

// ---- forward -------------------------------------------------------------------------------
// Grid of the two query-stationary kernels: one block per (pair of query blocks, GW query heads of a
// KV head, batch), pair index fastest.  A block runs query block `pair` and then its mirror image
// n-1-pair, so that under the causal mask every block sees the same number of key tiles; blocks that
// read the same K/V (one batch and KV head) are kept on one XCD.
struct QBlock {
    int pair, n_qblk, kvh, hgrp, b;
};
template <int GW>
__device__ __forceinline__ QBlock decode_qblock(const AttnArgs& a) {
    constexpr int QS = 4 / GW;
    QBlock r;
    r.n_qblk = (a.S + 32 * QS - 1) / (32 * QS);
    const int n_pairs = a.paired ? (r.n_qblk + 1) / 2 : r.n_qblk, groups = a.G / GW;
    // Blocks of one (batch, KV head) on one XCD.  Unpaired blocks differ in length under the causal mask: each XCD then
    // starts its longest ones first (pair index slowest in launch order), so that the short ones fill the end.
    int bid;
    const int per = gridDim.x / 8;
    if (!a.paired && gridDim.x % 8 == 0 && per % n_pairs == 0) {
        const int gx = per / n_pairs, xcd = blockIdx.x % 8, local = blockIdx.x / 8;  // gx groups of n_pairs blocks per XCD
        bid = (xcd * gx + local % gx) * n_pairs + local / gx;
    } else {
        bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    }
    r.pair = bid % n_pairs;
    const int y = (bid / n_pairs) % (a.Hkv * groups);
    r.kvh = y / groups;
    r.hgrp = y % groups;
    r.b = bid / (n_pairs * a.Hkv * groups);
    return r;
}

// TL: the kernel as it is plus time stamps (eisen_hip_attention_timeline)
template <int HD, int GW, bool TL = false>
__global__ __launch_bounds__(256) void fa_fwd_kernel(AttnArgs a) {
    constexpr int QS = 4 / GW, BKV = 64, KSTEPS = HD / 16, DT = HD / 32;
    __shared__ __attribute__((aligned(1024))) bf16_t Ksb[2][BKV * HD];  // swizzled tiles, see DirectTile
    __shared__ __attribute__((aligned(1024))) bf16_t Vsb[2][BKV * HD];
    const int lane = threadIdx.x & 63, g = lane >> 5, c = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int hsub = wave % GW, qsub = wave / GW;
    const QBlock blk = decode_qblock<GW>(a);
    const int kvh = blk.kvh, hq = kvh * a.G + blk.hgrp * GW + hsub, b = blk.b;
    const bf16_t* Qp = static_cast<const bf16_t*>(a.Q) + b * a.q_sb + hq * a.q_sh;
    const bf16_t* Kp = static_cast<const bf16_t*>(a.K) + b * a.k_sb + kvh * a.k_sh;
    const bf16_t* Vp = static_cast<const bf16_t*>(a.V) + b * a.k_sb + kvh * a.k_sh;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    DirectTile<HD, BKV, 4> kv_tile;
    kv_tile.init(a.k_ss, wave, lane);
    attn_stamp<TL>(a, 0, kStampStart, lane, wave);

    for (int pass = 0; pass < 2; pass++) {
        const int qblk = pass == 0 ? blk.n_qblk - 1 - blk.pair : blk.pair;  // the long one first
        if (pass == 1 && (!a.paired || qblk >= blk.n_qblk - 1 - blk.pair)) break;  // the middle block has no mirror
        if (pass == 1) __syncthreads();                                     // LDS tiles of the first pass are done with
        const int q0 = (qblk * QS + qsub) * 32, q = q0 + c;
        const bool valid_q = q < a.S;
        bf16x8 qf[KSTEPS];
#pragma unroll
        for (int st = 0; st < KSTEPS; st++)
            qf[st] = valid_q ? *reinterpret_cast<const bf16x8*>(Qp + (long long)q * a.q_ss + st * 16 + 8 * g) : zero8;
        f32x16 o[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[dt][v] = 0.f;
        // m is the reference point of the exponentials, not always the running maximum: it is only
        // moved when a row's maximum has grown by more than 2^8 since, which keeps every exponential
        // far inside the f32 and bf16 ranges and makes the rescaling of O rare.
        float m = -INFINITY, l = 0.f;

        const int block_qmax = min(a.S - 1, (qblk * QS + QS - 1) * 32 + 31);
        const int n_kt = a.causal ? block_qmax / BKV + 1 : (a.S + BKV - 1) / BKV;
        const int my_qmax = q0 < a.S ? q0 + 31 : -1;

        kv_tile.load_untracked(Kp, a.k_ss, 0, a.S, Ksb[0], wave, lane);
        kv_tile.load_untracked(Vp, a.k_ss, 0, a.S, Vsb[0], wave, lane);
        // The rows of Q have arrived before the tile loop: left pending, the compiler would wait for them at their first use
        // inside it, in every tile and for every load in flight, the prefetched tile's included.
#pragma unroll
        for (int st = 0; st < KSTEPS; st++) asm volatile("" : "+v"(qf[st]));
        // One 64-key tile.  MASKED is a compile-time flag: the tiles entirely below the diagonal and inside
        // the sequence run a loop body with no mask code and no branches at all.
        auto tile = [&](int kt, auto masked_c) {
            constexpr bool MASKED = decltype(masked_c)::value;
            const bf16_t* Ks = Ksb[kt & 1];
            const bf16_t* Vs = Vsb[kt & 1];
            wait_direct_loads();  // this wave's part of tile kt has landed
            __syncthreads();      // one barrier per tile: every wave is done with tile kt-1, whose buffer the next loads overwrite
            if (kt + 1 < n_kt) {
                kv_tile.load_untracked(Kp, a.k_ss, (kt + 1) * BKV, a.S, Ksb[(kt + 1) & 1], wave, lane);
                kv_tile.load_untracked(Vp, a.k_ss, (kt + 1) * BKV, a.S, Vsb[(kt + 1) & 1], wave, lane);
            }
            const int k0 = kt * BKV;
            if (my_qmax < 0 || (a.causal && k0 > my_qmax)) return;                // wave-uniform
            const bool two = !MASKED || (k0 + 32 < a.S && !(a.causal && k0 + 32 > my_qmax));  // the second 32 keys are visible
            f32x16 s[2];
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                for (int v = 0; v < 16; v++) s[sub][v] = sub == 0 ? 0.f : (two ? 0.f : -INFINITY);
                if (sub == 0 || two) {
#pragma unroll
                    for (int st = 0; st < KSTEPS; st++) {
                        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(Ks + tile_at<HD>(sub * 32 + c, st * 16 + 8 * g));
                        s[sub] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[st], s[sub], 0, 0, 0);
                    }
                }
            }
            // only tiles that touch the diagonal or the end of the sequence need the mask
            if (MASKED) {
                const int lim = min(a.causal ? q : a.S - 1, a.S - 1) - k0;  // tile rows above lim are masked
#pragma unroll
                for (int sub = 0; sub < 2; sub++)
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        if (sub * 32 + acc_row(v, g) > lim) s[sub][v] = -INFINITY;
            }
            // maximum of the raw scores (the positive scale is folded into the exponent's fma): four chains, not one of 16
            float mx4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
            for (int v = 0; v < 16; v++) mx4[v & 3] = fmaxf(mx4[v & 3], fmaxf(s[0][v], s[1][v]));
            float mx = fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3]));
            mx *= a.scale_log2e;
            // mx is the maximum over this lane's half of the tile's keys; the two lanes of a query exchange theirs only when
            // one of them has outgrown the reference point (then both take the same new one)
            if (__builtin_amdgcn_ballot_w64(mx > m + 8.0f) != 0) {
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const bool grow = mx > m + 8.0f;
                const float alpha = grow ? fast_exp2(m - mx) : 1.0f;
                m = grow ? mx : m;
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int v = 0; v < 16; v++) o[dt][v] *= alpha;
            }
            const float m_use = m == -INFINITY ? 0.f : m;
            float rs4[4] = {0.f, 0.f, 0.f, 0.f};  // four chains of eight additions, not one of 32
#pragma unroll
            for (int sub = 0; sub < 2; sub++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    s[sub][v] = fast_exp2(fmaf(s[sub][v], a.scale_log2e, -m_use));
                    rs4[v & 3] += s[sub][v];
                }
            const float rowsum = (rs4[0] + rs4[1]) + (rs4[2] + rs4[3]);
            l += rowsum;  // this lane's half of the row sum; the halves meet after the last tile
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                if (sub == 1 && !two) break;
                bf16x8 pf[2];
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int e = 0; e < 8; e++) pf[t][e] = (bf16_t)s[sub][8 * t + e];
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const bf16x8 vt = lds_tr_operand_swz<HD>(Vs, sub * 32, dt * 32, t, lane);
                        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vt, pf[t], o[dt], 0, 0, 0);
                    }
            }
        };
        // tiles [0, n_plain) need no mask for any query of this wave: all their keys are <= q0 and < S
        const int n_plain = min(n_kt, min(a.causal ? (q0 + 1) / BKV : n_kt, a.S / BKV));
        int kt = 0;
        attn_stamp<TL>(a, 0, kStampLoop + kStampsPerPass * pass, lane, wave);
        for (; kt < n_plain; kt++) tile(kt, std::false_type{});
        for (; kt < n_kt; kt++) tile(kt, std::true_type{});
        attn_stamp<TL>(a, 0, kStampLoopEnd + kStampsPerPass * pass, lane, wave);
        l += __shfl_xor(l, 32, 64);
        if (valid_q) {
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            bf16_t* Op = static_cast<bf16_t*>(a.Out) + b * a.q_sb + hq * a.q_sh + (long long)q * a.q_ss;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int vg = 0; vg < 4; vg++) {
                    bf16x4 w;
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = (bf16_t)(o[dt][vg * 4 + e] * inv);
                    *reinterpret_cast<bf16x4*>(Op + dt * 32 + 8 * vg + 4 * g) = w;
                }
            if (g == 0) a.LSE[((long long)b * a.Hq + hq) * a.S + q] = (m + log2f(l)) * kLn2;
        }
        attn_stamp<TL>(a, 0, kStampStored + kStampsPerPass * pass, lane, wave);
    }
}

// ---- backward: dQ (query-stationary); also writes D = rowsum(dO o O) for the dK/dV pass ------
// ABL: a part of the tile loop left out for a measurement (AttnAblation; kAblNone is the kernel)
//
// A block runs a long query block and then its short mirror image.  For head sizes up to 64 the two are one stream of
// K / V tiles through the two LDS buffers (the short block's first tile is requested under the long block's last one), and
// the rows of Q, dO and O of a wave's 32 queries arrive through three private LDS tiles of the wave, in whole rows; those of
// the short block are requested while the long block's tile loop runs, so that its start-up costs no trip to memory.
template <int HD, int GW, int ABL = kAblNone>
__global__ __launch_bounds__(256) void fa_bwd_dq_kernel(AttnArgs a) {
    constexpr int QS = 4 / GW, BKV = 64, KSTEPS = HD / 16, DT = HD / 32;
    constexpr bool STREAM = HD <= 64 && ABL != kAblTileLoads;
    constexpr int ROWS = 32 * HD;  // elements of a wave's Q, dO or O rows
    __shared__ __attribute__((aligned(1024))) bf16_t Ksb[2][BKV * HD];  // swizzled tiles, see DirectTile
    __shared__ __attribute__((aligned(1024))) bf16_t Vsb[2][BKV * HD];
    __shared__ __attribute__((aligned(1024))) bf16_t Rows[STREAM ? 4 * 3 * ROWS : 8];  // [wave][Q | dO | O], swizzled like the tiles
    const int lane = threadIdx.x & 63, g = lane >> 5, c = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int hsub = wave % GW, qsub = wave / GW;
    const QBlock blk = decode_qblock<GW>(a);
    const int kvh = blk.kvh, hq = kvh * a.G + blk.hgrp * GW + hsub, b = blk.b;
    const bf16_t* Kp = static_cast<const bf16_t*>(a.K) + b * a.k_sb + kvh * a.k_sh;
    const bf16_t* Vp = static_cast<const bf16_t*>(a.V) + b * a.k_sb + kvh * a.k_sh;
    const long long head_off = b * a.q_sb + hq * a.q_sh;
    const long long head_stat = ((long long)b * a.Hq + hq) * a.S;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    DirectTile<HD, BKV, 4> kv_tile;
    kv_tile.init(a.k_ss, wave, lane);
    DirectTile<HD, 32, 1> row_tile;
    if (STREAM) row_tile.init(a.q_ss, 0, lane);
    constexpr bool TL = ABL == kAblTimeline;
    attn_stamp<TL>(a, 1, kStampStart, lane, wave);
    bf16_t* my_rows = Rows + (STREAM ? wave * 3 * ROWS : 0);
    // the rows of Q, dO and O of this wave's queries of query block qb, straight into the wave's LDS tiles (rows past the
    // end repeat the last row; their queries get LSE = +inf below)
    auto request_rows = [&](int qb) {
        const int first = (qb * QS + qsub) * 32;
        row_tile.load_untracked(static_cast<const bf16_t*>(a.Q) + head_off, a.q_ss, first, a.S, my_rows, 0, lane);
        row_tile.load_untracked(static_cast<const bf16_t*>(a.dO) + head_off, a.q_ss, first, a.S, my_rows + ROWS, 0, lane);
        row_tile.load_untracked(static_cast<const bf16_t*>(a.O) + head_off, a.q_ss, first, a.S, my_rows + 2 * ROWS, 0, lane);
    };
    const int qblk_long = blk.n_qblk - 1 - blk.pair, qblk_short = blk.pair;
    const bool two = a.paired && qblk_short < qblk_long;  // the middle block has no mirror
    float lse_short = 0.f;  // STREAM: the short block's LSE, requested with the long block's
    if (STREAM) {
        kv_tile.load_untracked(Kp, a.k_ss, 0, a.S, Ksb[0], wave, lane);
        kv_tile.load_untracked(Vp, a.k_ss, 0, a.S, Vsb[0], wave, lane);
        request_rows(qblk_long);
        const int qs = (qblk_short * QS + qsub) * 32 + c;
        if (two && qs < a.S) lse_short = a.LSE[head_stat + qs];
    }
    int par = 0;  // STREAM: LDS buffer of the pass's first K / V tile

    for (int pass = 0; pass < 2; pass++) {
        const int qblk = pass == 0 ? qblk_long : qblk_short;
        if (pass == 1 && !two) break;
        const int q0 = (qblk * QS + qsub) * 32, q = q0 + c;
        const bool valid_q = q < a.S;
        const long long qoff = head_off + (long long)q * a.q_ss;
        const long long stat = head_stat + q;
        bf16x8 qf[KSTEPS], dof[KSTEPS];
        float dpart = 0.f, lse = 0.f;
        if (STREAM) {
            if (pass == 0) lse = valid_q ? a.LSE[stat] : 0.f;
            else lse = lse_short;
            wait_direct_loads();  // this wave's rows have landed (they are private to the wave: no barrier)
#pragma unroll
            for (int st = 0; st < KSTEPS; st++) {
                const int at = tile_at<HD>(c, st * 16 + 8 * g);
                qf[st] = *reinterpret_cast<const bf16x8*>(my_rows + at);
                dof[st] = *reinterpret_cast<const bf16x8*>(my_rows + ROWS + at);
                const bf16x8 of = *reinterpret_cast<const bf16x8*>(my_rows + 2 * ROWS + at);
#pragma unroll
                for (int e = 0; e < 8; e++) dpart += (float)dof[st][e] * (float)of[e];
            }
        } else {
            if (pass == 1) __syncthreads();
            // the first K / V tile travels with the rows of Q, dO and O, not behind the reduction that waits for them
            kv_tile.load_untracked(Kp, a.k_ss, 0, a.S, Ksb[0], wave, lane);
            kv_tile.load_untracked(Vp, a.k_ss, 0, a.S, Vsb[0], wave, lane);
#pragma unroll
            for (int st = 0; st < KSTEPS; st++) {
                const int d = st * 16 + 8 * g;
                qf[st] = valid_q ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.Q) + qoff + d) : zero8;
                dof[st] = valid_q ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.dO) + qoff + d) : zero8;
                const bf16x8 of = valid_q ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.O) + qoff + d) : zero8;
#pragma unroll
                for (int e = 0; e < 8; e++) dpart += (float)dof[st][e] * (float)of[e];
            }
            lse = valid_q ? a.LSE[stat] : 0.f;
        }
        const float Dq = dpart + __shfl_xor(dpart, 32, 64);
        const float lse2 = valid_q ? lse * kLog2e : INFINITY;
        if (valid_q && g == 0) {
            a.D[stat] = Dq;
            a.L2[stat] = -lse / a.scale;  // start value of the dK / dV kernel's score accumulators
        }

        f32x16 dq[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) dq[dt][v] = 0.f;

        const int block_qmax = min(a.S - 1, (qblk * QS + QS - 1) * 32 + 31);
        const int n_kt = a.causal ? block_qmax / BKV + 1 : (a.S + BKV - 1) / BKV;
        const int my_qmax = q0 < a.S ? q0 + 31 : -1;
        // STREAM, first pass: the short block's rows are requested under the second tile (the first one still shares the
        // memory system with every block's start-up), or under the only tile
        const int rows_at = pass == 0 && two ? min(1, n_kt - 1) : -1;

        auto tile = [&](int kt, auto masked_c) {
            constexpr bool MASKED = decltype(masked_c)::value;  // false: no key of the tile is masked for this wave
            const int buf = STREAM ? ((kt + par) & 1) : 0;
            const bf16_t* Ks = Ksb[ABL == kAblTileLoads ? 0 : (STREAM ? buf : (kt & 1))];
            const bf16_t* Vs = Vsb[ABL == kAblTileLoads ? 0 : (STREAM ? buf : (kt & 1))];
            wait_direct_loads();  // this wave's part of tile kt has landed
            __syncthreads();      // every wave is done with the tile before, whose buffer the next loads overwrite
            if (STREAM) {
                // the next tile of the stream: this pass's, or the first one of the short block
                const bool more = kt + 1 < n_kt;
                if (more || (pass == 0 && two)) {
                    const int first = more ? (kt + 1) * BKV : 0;
                    kv_tile.load_untracked(Kp, a.k_ss, first, a.S, Ksb[buf ^ 1], wave, lane);
                    kv_tile.load_untracked(Vp, a.k_ss, first, a.S, Vsb[buf ^ 1], wave, lane);
                }
                if (kt == rows_at) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the long block's rows have been read
                    request_rows(qblk_short);
                }
            } else if (ABL != kAblTileLoads && kt + 1 < n_kt) {
                kv_tile.load_untracked(Kp, a.k_ss, (kt + 1) * BKV, a.S, Ksb[(kt + 1) & 1], wave, lane);
                kv_tile.load_untracked(Vp, a.k_ss, (kt + 1) * BKV, a.S, Vsb[(kt + 1) & 1], wave, lane);
            }
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const int k0 = kt * BKV + sub * 32;
                if (MASKED && (k0 >= a.S || my_qmax < 0 || (a.causal && k0 > my_qmax))) continue;
                f32x16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = -Dq; }  // the MFMA chain delivers dP - D
#pragma unroll
                for (int st = 0; st < KSTEPS; st++) {
                    const bf16x8 kf = ABL == kAblOperandReads ? dof[st] : *reinterpret_cast<const bf16x8*>(Ks + tile_at<HD>(sub * 32 + c, st * 16 + 8 * g));
                    const bf16x8 vf = ABL == kAblOperandReads ? qf[st] : *reinterpret_cast<const bf16x8*>(Vs + tile_at<HD>(sub * 32 + c, st * 16 + 8 * g));
                    if (ABL == kAblScoreMfmas) {
                        s[st] += (float)kf[0];
                        dp[st] += (float)vf[0];
                    } else {
                        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[st], s, 0, 0, 0);
                        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, dof[st], dp, 0, 0, 0);
                    }
                }
                bf16x8 dsf[2];
                // a query past the end has LSE = +inf; keys past the end (their tile rows repeat the last
                // key) and keys above the causal diagonal are masked
                float p[16];
#pragma unroll
                for (int v = 0; v < 16; v++) p[v] = ABL == kAblSoftmax ? s[v] : fast_exp2(fmaf(s[v], a.scale_log2e, -lse2));
                if (MASKED && ((a.causal && k0 + 31 > q0) || k0 + 32 > a.S)) {
                    const int rel = min(a.causal ? q : a.S - 1, a.S - 1) - k0;  // keys k0 + row > rel are masked
#pragma unroll
                    for (int v = 0; v < 16; v++)
                        if (acc_row(v, g) > rel) p[v] = 0.f;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) dsf[v >> 3][v & 7] = (bf16_t)(ABL == kAblSoftmax ? dp[v] : p[v] * dp[v]);
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const bf16x8 ktr = ABL == kAblTransposedReads ? qf[dt * 2 + t] : lds_tr_operand_swz<HD>(Ks, sub * 32, dt * 32, t, lane);
                        if (ABL == kAblSecondMfmas) dq[dt][0] += (float)ktr[0] * (float)dsf[t][0];
                        else dq[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktr, dsf[t], dq[dt], 0, 0, 0);
                    }
            }
        };
        const int n_plain = my_qmax < 0 ? 0 : min(n_kt, min(a.causal ? (q0 + 1) / BKV : n_kt, a.S / BKV));
        int kt = 0;
        attn_stamp<TL>(a, 1, kStampLoop + kStampsPerPass * pass, lane, wave);
        for (; kt < n_plain; kt++) tile(kt, std::false_type{});
        for (; kt < n_kt; kt++) tile(kt, std::true_type{});
        attn_stamp<TL>(a, 1, kStampLoopEnd + kStampsPerPass * pass, lane, wave);
        par = (par + n_kt) & 1;
        if (valid_q) {
            bf16_t* dQp = static_cast<bf16_t*>(a.dQ) + qoff;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int vg = 0; vg < 4; vg++) {
                    float x[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] = dq[dt][vg * 4 + e] * a.scale;
                    if (a.rope) unrotate_pairs<2>(x, a.rope + (size_t)q * (HD / 2) + (dt * 32 + 8 * vg + 4 * g) / 2);
                    bf16x4 w;
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = (bf16_t)x[e];
                    *reinterpret_cast<bf16x4*>(dQp + dt * 32 + 8 * vg + 4 * g) = w;
                }
        }
        attn_stamp<TL>(a, 1, kStampStored + kStampsPerPass * pass, lane, wave);
    }
}

// ---- backward: dK, dV (key-stationary, summed over the query heads of the group) -------------
// One block owns the keys of two 32-key blocks of one KV head, a heavy one and its light mirror image
// under the causal mask, so every block of the grid has the same amount of work.  Its four waves
// each take every fourth (query head of the group, 32-query tile) item, with a private LDS tile and
// no block barrier inside the item loop; their partial dK/dV are summed through LDS once per key block.
template <int HD>
__global__ __launch_bounds__(256) void fa_bwd_dkv_kernel(AttnArgs a) {
    constexpr int PITCH = HD + 8, KSTEPS = HD / 16, DT = HD / 32, TILE = 32 * PITCH;
    constexpr int CPR = HD / 8, CH = 32 * CPR / 64;  // 16-byte chunks per row / per lane of a tile
    __shared__ __attribute__((aligned(16))) bf16_t tiles[4][2][TILE];  // per wave: Q tile, dO tile
    __shared__ __attribute__((aligned(16))) float stats[4][64];        // per wave: LSE*log2(e) | D
    static_assert(2 * TILE * sizeof(bf16_t) >= 32 * HD * sizeof(float), "reduction scratch reuses the tiles");
    const int lane = threadIdx.x & 63, g = lane >> 5, c = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_qt = (a.S + 31) / 32;
    // grid: x = key-block pair, fastest; then KV head, then batch.  Blocks of one (batch, KV head) read
    // the same Q/dO tiles, so they are kept on one XCD.
    const int n_pairs = (n_qt + 1) / 2;
    const int bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int pair = bid % n_pairs, kvh = (bid / n_pairs) % a.Hkv, b = bid / (n_pairs * a.Hkv);
    bf16_t* Qs = tiles[wave][0];
    bf16_t* dOs = tiles[wave][1];
    float* st = stats[wave];
    float* red = reinterpret_cast<float*>(tiles[wave][0]);
    const bf16_t* Qg = static_cast<const bf16_t*>(a.Q) + b * a.q_sb;
    const bf16_t* dOg = static_cast<const bf16_t*>(a.dO) + b * a.q_sb;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const float* stat_src = g == 0 ? a.LSE : a.D;  // lanes 0-31 fetch the tile's LSE, lanes 32-63 its D
    int loff[CH];  // element offset of this lane's chunk i inside a 32-row Q / dO tile
#pragma unroll
    for (int i = 0; i < CH; i++) loff[i] = ((i * 64 + lane) / CPR) * (int)a.q_ss + ((i * 64 + lane) % CPR) * 8;

    for (int pass = 0; pass < 2; pass++) {
        const int kb = pass == 0 ? pair : n_qt - 1 - pair;
        if (pass == 1 && kb <= pair) break;  // odd block count: the middle block has no mirror
        const int k0 = kb * 32, key = k0 + c;
        const bool valid_k = key < a.S;
        const long long koff = b * a.k_sb + kvh * a.k_sh + (long long)key * a.k_ss;
        bf16x8 kf[KSTEPS], vf[KSTEPS];
#pragma unroll
        for (int st_ = 0; st_ < KSTEPS; st_++) {
            const int d = st_ * 16 + 8 * g;
            kf[st_] = valid_k ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.K) + koff + d) : zero8;
            vf[st_] = valid_k ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.V) + koff + d) : zero8;
        }
        f32x16 dk[DT], dv[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) { dk[dt][v] = 0.f; dv[dt][v] = 0.f; }

        const int qt_start = a.causal ? kb : 0;  // the diagonal tile is the first one that sees these keys
        const int per_head = n_qt - qt_start;
        const int n_items = a.G * per_head;      // (query head of the group, query tile), head-major

        bf16x8 rq[CH], rdo[CH];
        float rstat = 0.f;
        auto fetch = [&](int item) {
            const int hq = kvh * a.G + item / per_head, q0 = (qt_start + item % per_head) * 32;
            // wave-uniform tile origin in scalar registers; the per-lane part of every address is loff / c
            const bf16_t* qp = Qg + hq * a.q_sh + (long long)q0 * a.q_ss;
            const bf16_t* dop = dOg + hq * a.q_sh + (long long)q0 * a.q_ss;
            const long long si = ((long long)b * a.Hq + hq) * a.S + q0;
            if (q0 + 32 <= a.S) {
#pragma unroll
                for (int i = 0; i < CH; i++) {
                    rq[i] = *reinterpret_cast<const bf16x8*>(qp + loff[i]);
                    rdo[i] = *reinterpret_cast<const bf16x8*>(dop + loff[i]);
                }
                rstat = stat_src[si + c];  // raw: any arithmetic here would wait for the load on the spot
            } else {
#pragma unroll
                for (int i = 0; i < CH; i++) {
                    const bool ok = q0 + (i * 64 + lane) / CPR < a.S;
                    rq[i] = ok ? *reinterpret_cast<const bf16x8*>(qp + loff[i]) : zero8;
                    rdo[i] = ok ? *reinterpret_cast<const bf16x8*>(dop + loff[i]) : zero8;
                }
                // a query past the end gets LSE = +inf, so its probabilities come out as exactly zero
                rstat = q0 + c < a.S ? stat_src[si + c] : (g == 0 ? INFINITY : 0.f);
            }
        };
        if (wave < n_items) fetch(wave);
        for (int item = wave; item < n_items; item += 4) {
            // The tile is private to the wave and LDS serves a wave's requests in order, so the stores
            // below cannot overtake the previous item's reads; the fences keep the compiler from
            // moving accesses of other lanes' data across them.
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
            for (int i = 0; i < CH; i++) {
                const int ch = i * 64 + lane;
                *reinterpret_cast<bf16x8*>(Qs + (ch / CPR) * PITCH + (ch % CPR) * 8) = rq[i];
                *reinterpret_cast<bf16x8*>(dOs + (ch / CPR) * PITCH + (ch % CPR) * 8) = rdo[i];
            }
            st[lane] = g == 0 ? rstat * kLog2e : rstat;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (item + 4 < n_items) fetch(item + 4);

            f32x16 s, dp;
#pragma unroll
            for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
            for (int st_ = 0; st_ < KSTEPS; st_++) {
                const bf16x8 qa = *reinterpret_cast<const bf16x8*>(Qs + c * PITCH + st_ * 16 + 8 * g);
                const bf16x8 da = *reinterpret_cast<const bf16x8*>(dOs + c * PITCH + st_ * 16 + 8 * g);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[st_], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vf[st_], dp, 0, 0, 0);
            }
            bf16x8 pf[2], dsf[2];
            float p[16];
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const float4 l4 = *reinterpret_cast<const float4*>(st + 8 * vg + 4 * g);
                const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) p[vg * 4 + e] = fast_exp2(fmaf(s[vg * 4 + e], a.scale_log2e, -lv[e]));
            }
            // only the diagonal tile is cut by the causal mask; rows and keys past the end need no
            // mask (zero probability through LSE = +inf, respectively never stored)
            if (a.causal && (item % per_head) == 0) {
                asm volatile("" ::: "memory");  // keeps this a branch taken once per head, not 16 selects per tile
#pragma unroll
                for (int v = 0; v < 16; v++)
                    if (c > acc_row(v, g)) p[v] = 0.f;  // key k0+c is after query q0+row
            }
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const float4 d4 = *reinterpret_cast<const float4*>(st + 32 + 8 * vg + 4 * g);
                const float dvv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int v = vg * 4 + e;
                    pf[v >> 3][v & 7] = (bf16_t)p[v];
                    dsf[v >> 3][v & 7] = (bf16_t)(p[v] * (dp[v] - dvv[e]));
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const bf16x8 dotr = lds_tr_operand(dOs, PITCH, 0, dt * 32, t, lane);
                    const bf16x8 qtr = lds_tr_operand(Qs, PITCH, 0, dt * 32, t, lane);
                    dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[t], dotr, dv[dt], 0, 0, 0);
                    dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[t], qtr, dk[dt], 0, 0, 0);
                }
        }

        // Sum the four waves' partial results, dK then dV, through the (now idle) tile memory.
        bf16_t* outs[2] = {static_cast<bf16_t*>(a.dK) + b * a.k_sb + kvh * a.k_sh,
                           static_cast<bf16_t*>(a.dV) + b * a.k_sb + kvh * a.k_sh};
#pragma unroll
        for (int which = 0; which < 2; which++) {
            __syncthreads();  // every wave is done with its tile / with the previous reduction
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    red[acc_row(v, g) * HD + dt * 32 + c] = which == 0 ? dk[dt][v] * a.scale : dv[dt][v];
            __syncthreads();
            // 32 x HD outputs, 8 consecutive ones per thread step
            for (int e0 = threadIdx.x * 8; e0 < 32 * HD; e0 += 256 * 8) {
                float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const float* src = reinterpret_cast<const float*>(tiles[w][0]) + e0;
                    const float4 x0 = *reinterpret_cast<const float4*>(src);
                    const float4 x1 = *reinterpret_cast<const float4*>(src + 4);
                    acc8[0] += x0.x; acc8[1] += x0.y; acc8[2] += x0.z; acc8[3] += x0.w;
                    acc8[4] += x1.x; acc8[5] += x1.y; acc8[6] += x1.z; acc8[7] += x1.w;
                }
                const int kr = k0 + e0 / HD;
                if (kr < a.S) {
                    if (which == 0 && a.rope) unrotate_pairs<4>(acc8, a.rope + (size_t)kr * (HD / 2) + (e0 % HD) / 2);
                    bf16x8 o8;
#pragma unroll
                    for (int e = 0; e < 8; e++) o8[e] = (bf16_t)acc8[e];
                    *reinterpret_cast<bf16x8*>(outs[which] + (long long)kr * a.k_ss + e0 % HD) = o8;
                }
            }
        }
        __syncthreads();  // the reduction's reads are over before the next pass refills the tiles
    }
}

// ---- f32 path: one wave per row, any head_dim ---------------------------------------------------
// forward: scores in LDS (S floats), same arithmetic as the unfused chain
// (bmm -> *scale -> mask -> softmax -> bmm; src/nn/attention.rs:338-375).
__global__ __launch_bounds__(64) void attn_f32_fwd_kernel(AttnArgs a) {
    extern __shared__ float sc[];
    const int q = blockIdx.x, hq = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int kvh = hq / a.G;
    const float* Qr = static_cast<const float*>(a.Q) + b * a.q_sb + hq * a.q_sh + (long long)q * a.q_ss;
    const float* Kp = static_cast<const float*>(a.K) + b * a.k_sb + kvh * a.k_sh;
    const float* Vp = static_cast<const float*>(a.V) + b * a.k_sb + kvh * a.k_sh;
    const int nk = a.causal ? q + 1 : a.S;
    float mx = -INFINITY;
    for (int j = lane; j < nk; j += 64) {
        const float* Kr = Kp + (long long)j * a.k_ss;
        float dot = 0.f;
        for (int d = 0; d < a.hd; d++) dot += Qr[d] * Kr[d];
        dot *= a.scale;
        sc[j] = dot;
        mx = fmaxf(mx, dot);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lane; j < nk; j += 64) {
        const float e = __expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    __syncthreads();
    float* Or = static_cast<float*>(a.Out) + b * a.q_sb + hq * a.q_sh + (long long)q * a.q_ss;
    for (int d = lane; d < a.hd; d += 64) {
        float acc = 0.f;
        for (int j = 0; j < nk; j++) acc += sc[j] * Vp[(long long)j * a.k_ss + d];
        Or[d] = acc / sum;
    }
    if (lane == 0) a.LSE[((long long)b * a.Hq + hq) * a.S + q] = mx + logf(sum);
}

__global__ __launch_bounds__(64) void attn_f32_bwd_dq_kernel(AttnArgs a) {
    extern __shared__ float ds[];
    const int q = blockIdx.x, hq = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int kvh = hq / a.G;
    const long long qoff = b * a.q_sb + hq * a.q_sh + (long long)q * a.q_ss;
    const float* Qr = static_cast<const float*>(a.Q) + qoff;
    const float* dOr = static_cast<const float*>(a.dO) + qoff;
    const float* Or = static_cast<const float*>(a.O) + qoff;
    const float* Kp = static_cast<const float*>(a.K) + b * a.k_sb + kvh * a.k_sh;
    const float* Vp = static_cast<const float*>(a.V) + b * a.k_sb + kvh * a.k_sh;
    const long long stat = ((long long)b * a.Hq + hq) * a.S + q;
    float dpart = 0.f;
    for (int d = lane; d < a.hd; d += 64) dpart += dOr[d] * Or[d];
    const float Dq = wave_sum(dpart);
    if (lane == 0) a.D[stat] = Dq;
    const float lse = a.LSE[stat];
    const int nk = a.causal ? q + 1 : a.S;
    for (int j = lane; j < nk; j += 64) {
        const float* Kr = Kp + (long long)j * a.k_ss;
        const float* Vr = Vp + (long long)j * a.k_ss;
        float dot = 0.f, dp = 0.f;
        for (int d = 0; d < a.hd; d++) {
            dot += Qr[d] * Kr[d];
            dp += dOr[d] * Vr[d];
        }
        const float p = __expf(dot * a.scale - lse);
        ds[j] = p * (dp - Dq) * a.scale;
    }
    __syncthreads();
    float* dQr = static_cast<float*>(a.dQ) + qoff;
    for (int d = lane; d < a.hd; d += 64) {
        float acc = 0.f;
        for (int j = 0; j < nk; j++) acc += ds[j] * Kp[(long long)j * a.k_ss + d];
        dQr[d] = acc;
    }
}

// one wave per key row; walks the query heads of the group (ascending, like repeat_kv's
// backward) and the queries that see this key.
__global__ __launch_bounds__(64) void attn_f32_bwd_dkv_kernel(AttnArgs a) {
    extern __shared__ float sm[];  // p[S], ds[S]
    float* pbuf = sm;
    float* dsbuf = sm + a.S;
    const int j = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const long long koff = b * a.k_sb + kvh * a.k_sh + (long long)j * a.k_ss;
    const float* Kr = static_cast<const float*>(a.K) + koff;
    const float* Vr = static_cast<const float*>(a.V) + koff;
    const int qs = a.causal ? j : 0;
    // per-lane accumulators for d = lane, lane+64, ... (head_dim <= 256)
    float accK[4] = {0.f, 0.f, 0.f, 0.f}, accV[4] = {0.f, 0.f, 0.f, 0.f};
    for (int hh = 0; hh < a.G; hh++) {
        const int hq = kvh * a.G + hh;
        const float* Qp = static_cast<const float*>(a.Q) + b * a.q_sb + hq * a.q_sh;
        const float* dOp = static_cast<const float*>(a.dO) + b * a.q_sb + hq * a.q_sh;
        const long long stat0 = ((long long)b * a.Hq + hq) * a.S;
        __syncthreads();
        for (int q = qs + lane; q < a.S; q += 64) {
            const float* Qr = Qp + (long long)q * a.q_ss;
            const float* dOr = dOp + (long long)q * a.q_ss;
            float dot = 0.f, dp = 0.f;
            for (int d = 0; d < a.hd; d++) {
                dot += Qr[d] * Kr[d];
                dp += dOr[d] * Vr[d];
            }
            const float p = __expf(dot * a.scale - a.LSE[stat0 + q]);
            pbuf[q] = p;
            dsbuf[q] = p * (dp - a.D[stat0 + q]) * a.scale;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int d = lane + 64 * u;
            if (d < a.hd)
                for (int q = qs; q < a.S; q++) {
                    accV[u] += pbuf[q] * dOp[(long long)q * a.q_ss + d];
                    accK[u] += dsbuf[q] * Qp[(long long)q * a.q_ss + d];
                }
        }
    }
    float* dKr = static_cast<float*>(a.dK) + koff;
    float* dVr = static_cast<float*>(a.dV) + koff;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int d = lane + 64 * u;
        if (d < a.hd) {
            dKr[d] = accK[u];
            dVr[d] = accV[u];
        }
    }
}

int fill_args(eisen_ctx* ctx, AttnArgs& a, int dtype, size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
              const long long* q_strides, const long long* kv_strides, float scale, int causal, const char* who) {
    EISEN_REQUIRE(ctx, eisen_dtype_ok(dtype), EISEN_E_ARG, "%s: unknown dtype %d", who, dtype);
    EISEN_REQUIRE(ctx, B > 0 && S > 0 && Hq > 0 && Hkv > 0 && hd > 0, EISEN_E_SHAPE, "%s: empty dimension", who);
    EISEN_REQUIRE(ctx, Hq % Hkv == 0, EISEN_E_SHAPE, "%s: %zu query heads not divisible by %zu kv heads", who, Hq, Hkv);
    EISEN_REQUIRE(ctx, B < 65536 && Hq < 65536 && S < (size_t(1) << 24) && hd <= 256, EISEN_E_SHAPE, "%s: dimension out of range", who);
    if (dtype == EISEN_BF16)
        EISEN_REQUIRE(ctx, hd == 32 || hd == 64 || hd == 128, EISEN_E_SHAPE, "%s: bf16 path supports head_dim 32, 64, 128 (got %zu)", who, hd);
    a.B = (int)B; a.S = (int)S; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.G = (int)(Hq / Hkv); a.hd = (int)hd;
    if (q_strides) { a.q_sb = q_strides[0]; a.q_ss = q_strides[1]; a.q_sh = q_strides[2]; }
    else { a.q_sb = (long long)(S * Hq * hd); a.q_ss = (long long)(Hq * hd); a.q_sh = (long long)hd; }
    if (kv_strides) { a.k_sb = kv_strides[0]; a.k_ss = kv_strides[1]; a.k_sh = kv_strides[2]; }
    else { a.k_sb = (long long)(S * Hkv * hd); a.k_ss = (long long)(Hkv * hd); a.k_sh = (long long)hd; }
    if (dtype == EISEN_BF16)
        EISEN_REQUIRE(ctx, a.q_sb % 8 == 0 && a.q_ss % 8 == 0 && a.q_sh % 8 == 0 && a.k_sb % 8 == 0 && a.k_ss % 8 == 0 && a.k_sh % 8 == 0,
                      EISEN_E_ALIGN, "%s: strides must be multiples of 8 elements for bf16", who);
    // the key-stationary backward starts its score accumulators at -LSE / scale; a softmax scale is positive anyway
    EISEN_REQUIRE(ctx, std::isfinite(scale) && scale >= 1e-30f && scale <= 1e30f, EISEN_E_ARG, "%s: softmax scale %g is not a positive finite number", who, (double)scale);
    a.scale = scale;
    a.scale_log2e = scale * kLog2e;
    a.causal = causal;
    return 0;
}

// Algorithmic flops of one attention GEMM over the visible (query, key) pairs.
static double attn_pair_flops(const AttnArgs& a) {
    const double pairs = a.causal ? (double)a.S * ((double)a.S + 1.0) / 2.0 : (double)a.S * (double)a.S;
    return 2.0 * (double)a.hd * pairs * (double)a.B * (double)a.Hq;
}

template <int HD>
void launch_fwd(eisen_ctx* ctx, AttnArgs a) {
    EisenProfScope prof(ctx, "attn_fwd_bf16", 2.0 * attn_pair_flops(a), true);
    const int gw = a.G % 4 == 0 ? 4 : (a.G % 2 == 0 ? 2 : 1);
    const int qs = 4 / gw;
    const int n_qblk = eisen_ceil_div(a.S, 32 * qs), per_q = a.Hkv * (a.G / gw) * a.B;
    // One block per query block, the long ones launched first (decode_qblock): blocks that finish early take the next one,
    // which evens out more than pairing long with short blocks does.  Pairing remains for grids that cannot be ordered so.
    const long long blocks = (long long)n_qblk * per_q;
    a.paired = a.causal && blocks >= 1024 && !(blocks % 8 == 0 && (blocks / 8) % n_qblk == 0);
    dim3 grid((unsigned)((a.paired ? (n_qblk + 1) / 2 : n_qblk) * per_q));
    if (HD == 64 && gw == 4 && a.stamps) fa_fwd_kernel<64, 4, true><<<grid, 256, 0, ctx->stream>>>(a);
    else if (gw == 4) fa_fwd_kernel<HD, 4><<<grid, 256, 0, ctx->stream>>>(a);
    else if (gw == 2) fa_fwd_kernel<HD, 2><<<grid, 256, 0, ctx->stream>>>(a);
    else fa_fwd_kernel<HD, 1><<<grid, 256, 0, ctx->stream>>>(a);
}
template <int HD>
void launch_bwd(eisen_ctx* ctx, AttnArgs a) {
    const int gw = a.G % 4 == 0 ? 4 : (a.G % 2 == 0 ? 2 : 1);
    const int qs = 4 / gw;
    const int n_qblk = eisen_ceil_div(a.S, 32 * qs), per_q = a.Hkv * (a.G / gw) * a.B;
    // pairing long and short query blocks balances the causal mask; it is only worth halving the
    // number of blocks when at least two per CU remain
    a.paired = a.causal && (long long)n_qblk * per_q >= 1024;
    dim3 grid((unsigned)((a.paired ? (n_qblk + 1) / 2 : n_qblk) * per_q));
    {   // dQ = scale dS K: one of the four backward GEMMs (S and dP are recomputed here as well)
        EisenProfScope prof(ctx, "attn_bwd_dq_bf16", 1.0 * attn_pair_flops(a), true);
        if (HD == 64 && gw == 4 && a.ablation != kAblNone) {  // measurement runs, at the shape the measurements are quoted for
            switch (a.ablation) {
                case kAblTransposedReads: fa_bwd_dq_kernel<64, 4, kAblTransposedReads><<<grid, 256, 0, ctx->stream>>>(a); break;
                case kAblOperandReads: fa_bwd_dq_kernel<64, 4, kAblOperandReads><<<grid, 256, 0, ctx->stream>>>(a); break;
                case kAblSecondMfmas: fa_bwd_dq_kernel<64, 4, kAblSecondMfmas><<<grid, 256, 0, ctx->stream>>>(a); break;
                case kAblTileLoads: fa_bwd_dq_kernel<64, 4, kAblTileLoads><<<grid, 256, 0, ctx->stream>>>(a); break;
                case kAblSoftmax: fa_bwd_dq_kernel<64, 4, kAblSoftmax><<<grid, 256, 0, ctx->stream>>>(a); break;
                case kAblTimeline: fa_bwd_dq_kernel<64, 4, kAblTimeline><<<grid, 256, 0, ctx->stream>>>(a); break;
                default: fa_bwd_dq_kernel<64, 4, kAblScoreMfmas><<<grid, 256, 0, ctx->stream>>>(a); break;
            }
        } else if (gw == 4) fa_bwd_dq_kernel<HD, 4><<<grid, 256, 0, ctx->stream>>>(a);
        else if (gw == 2) fa_bwd_dq_kernel<HD, 2><<<grid, 256, 0, ctx->stream>>>(a);
        else fa_bwd_dq_kernel<HD, 1><<<grid, 256, 0, ctx->stream>>>(a);
    }
    const int n_kb = eisen_ceil_div(a.S, 32);  // 32-key blocks, handled in heavy/light pairs
    dim3 grid2((unsigned)((n_kb + 1) / 2 * a.Hkv * a.B));
    {   // dP, dV, dK: three of the four backward GEMMs
        EisenProfScope prof(ctx, "attn_bwd_dkv_bf16", 3.0 * attn_pair_flops(a), true);
        if (HD <= 64 && eisen_attention_dkv32_supports(a)) eisen_attention_launch_dkv32(ctx, a);
        else fa_bwd_dkv_kernel<HD><<<grid2, 256, 0, ctx->stream>>>(a);
    }
}

}  // namespace

extern "C" int eisen_hip_attention_forward(eisen_ctx* ctx, const void* q, const void* k, const void* v, void* out,
                                           float* lse, int dtype, size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
                                           const long long* q_strides, const long long* kv_strides, float scale,
                                           int causal) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, q && k && v && out && lse, EISEN_E_ARG, "attention_forward: null pointer");
    AttnArgs a{};
    int rc = fill_args(ctx, a, dtype, B, S, Hq, Hkv, hd, q_strides, kv_strides, scale, causal, "attention_forward");
    if (rc) return rc;
    a.Q = q; a.K = k; a.V = v; a.Out = out; a.LSE = lse;
    a.stamps = ctx->attn_stamps;
    a.stamp_waves = ctx->attn_stamp_waves;
    if (dtype == EISEN_BF16) {
        EISEN_REQUIRE(ctx, eisen_aligned(q, 16) && eisen_aligned(k, 16) && eisen_aligned(v, 16) && eisen_aligned(out, 16),
                      EISEN_E_ALIGN, "attention_forward: bf16 buffers must be 16-byte aligned");
        if (hd == 32) launch_fwd<32>(ctx, a);
        else if (hd == 64) launch_fwd<64>(ctx, a);
        else launch_fwd<128>(ctx, a);
    } else {
        EISEN_REQUIRE(ctx, S * sizeof(float) <= 64 * 1024, EISEN_E_SHAPE, "attention_forward: f32 path supports S <= 16384");
        dim3 grid((unsigned)S, (unsigned)Hq, (unsigned)B);
        attn_f32_fwd_kernel<<<grid, 64, S * sizeof(float), ctx->stream>>>(a);
    }
    EISEN_LAUNCH_CHECK(ctx, "attention forward");
    return 0;
}

extern "C" int eisen_hip_attention_ablation(eisen_ctx* ctx, int part) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, part >= 0 && part < kAblCount, EISEN_E_ARG, "attention_ablation: part %d outside [0, %d)", part, (int)kAblCount);
    ctx->attn_ablation = part;
    return 0;
}

extern "C" int eisen_hip_attention_timeline(eisen_ctx* ctx, long long* stamps, size_t waves) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, (stamps == nullptr) == (waves == 0), EISEN_E_ARG, "attention_timeline: a buffer and a wave count come together (or neither)");
    EISEN_REQUIRE(ctx, waves <= (size_t(1) << 24), EISEN_E_ARG, "attention_timeline: %zu waves is beyond 2^24", waves);
    EISEN_REQUIRE(ctx, eisen_aligned(stamps, 8), EISEN_E_ALIGN, "attention_timeline: the buffer must be 8-byte aligned");
    ctx->attn_stamps = stamps;
    ctx->attn_stamp_waves = (int)waves;
    return 0;
}

int eisen_attention_scratch_init(eisen_ctx* ctx) {
    EISEN_REQUIRE(ctx, ctx->device >= 0 && ctx->device < kMaxDevices, EISEN_E_ARG, "device index %d beyond the %d this library keeps scratch for", ctx->device, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_attn_bwd_scratch_mu);
    if (!g_attn_bwd_scratch_done[ctx->device]) {
        EISEN_HIP_TRY(ctx, hipSetDevice(ctx->device));
        EISEN_HIP_TRY(ctx, hipEventCreateWithFlags(&g_attn_bwd_scratch_done[ctx->device], hipEventDisableTiming));
    }
    if (!g_attn_bwd_scratch_ptr[ctx->device]) {
        float* p = nullptr;
        EISEN_HIP_TRY(ctx, hipSetDevice(ctx->device));
        EISEN_HIP_TRY(ctx, hipGetSymbolAddress((void**)&p, HIP_SYMBOL(g_attn_bwd_scratch)));
        EISEN_REQUIRE(ctx, p != nullptr, EISEN_E_STATE, "hipGetSymbolAddress returned a null address for the attention scratch");
        g_attn_bwd_scratch_ptr[ctx->device] = p;
    }
    ctx->attn_scratch = g_attn_bwd_scratch_ptr[ctx->device];
    return 0;
}

// scratch: where D = rowsum(dO o O) goes; nullptr = the context's grow-only workspace
static int attention_backward_common(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                     const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype,
                                     size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
                                     const long long* q_strides, const long long* kv_strides, float scale,
                                     int causal, bool rope, float* scratch = nullptr) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, q && k && v && out && dout && lse && dq && dk && dv, EISEN_E_ARG, "attention_backward: null pointer");
    AttnArgs a{};
    int rc = fill_args(ctx, a, dtype, B, S, Hq, Hkv, hd, q_strides, kv_strides, scale, causal, "attention_backward");
    if (rc) return rc;
    a.Q = q; a.K = k; a.V = v; a.O = out; a.dO = dout; a.LSE = const_cast<float*>(lse);
    a.dQ = dq; a.dK = dk; a.dV = dv;
    a.ablation = ctx->attn_ablation;
    a.stamps = ctx->attn_stamps;
    a.stamp_waves = ctx->attn_stamp_waves;
    if (a.stamps && a.ablation == kAblNone) a.ablation = kAblTimeline;
    if (scratch) {
        a.D = scratch;
    } else {
        void* ws = nullptr;
        rc = eisen_workspace(ctx, 2 * B * Hq * S * sizeof(float), &ws);
        if (rc) return rc;
        a.D = static_cast<float*>(ws);
    }
    a.L2 = a.D + B * Hq * S;
    if (rope) {
        rc = eisen_rope_table_get(ctx, S, hd, &a.rope);
        if (rc) return rc;
    }
    if (dtype == EISEN_BF16) {
        EISEN_REQUIRE(ctx, eisen_aligned(q, 16) && eisen_aligned(k, 16) && eisen_aligned(v, 16) && eisen_aligned(out, 16) &&
                               eisen_aligned(dout, 16) && eisen_aligned(dq, 16) && eisen_aligned(dk, 16) && eisen_aligned(dv, 16),
                      EISEN_E_ALIGN, "attention_backward: bf16 buffers must be 16-byte aligned");
        if (hd == 32) launch_bwd<32>(ctx, a);
        else if (hd == 64) launch_bwd<64>(ctx, a);
        else launch_bwd<128>(ctx, a);
    } else {
        EISEN_REQUIRE(ctx, 2 * S * sizeof(float) <= 64 * 1024, EISEN_E_SHAPE, "attention_backward: f32 path supports S <= 8192");
        dim3 grid((unsigned)S, (unsigned)Hq, (unsigned)B);
        attn_f32_bwd_dq_kernel<<<grid, 64, S * sizeof(float), ctx->stream>>>(a);
        dim3 grid2((unsigned)S, (unsigned)Hkv, (unsigned)B);
        attn_f32_bwd_dkv_kernel<<<grid2, 64, 2 * S * sizeof(float), ctx->stream>>>(a);
    }
    EISEN_LAUNCH_CHECK(ctx, "attention backward");
    return 0;
}

extern "C" int eisen_hip_attention_backward(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                            const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype,
                                            size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
                                            const long long* q_strides, const long long* kv_strides, float scale,
                                            int causal) {
    return attention_backward_common(ctx, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, q_strides, kv_strides, scale, causal, false);
}

extern "C" int eisen_hip_attention_backward_noalloc(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                                    const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype,
                                                    size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd,
                                                    const long long* q_strides, const long long* kv_strides, float scale,
                                                    int causal) {
    EISEN_CHECK_CTX(ctx);
    EISEN_REQUIRE(ctx, ctx->attn_scratch != nullptr, EISEN_E_STATE, "attention_backward_noalloc: the context has no scratch address");
    EISEN_REQUIRE(ctx, B > 0 && S > 0 && Hq > 0 && B <= kNoAllocMaxRows && S <= kNoAllocMaxRows && Hq <= kNoAllocMaxRows &&
                           B * Hq <= kNoAllocMaxRows && B * Hq * S <= kNoAllocMaxRows,
                  EISEN_E_SHAPE, "attention_backward_noalloc: batch * query heads * seq = %zu * %zu * %zu exceeds the %zu rows of the fixed scratch",
                  B, Hq, S, kNoAllocMaxRows);
    // Calls that share this GPU's array run one after the other: this call's stream first waits for the kernels of the
    // previous one, on whatever context or stream that was.  A stream under graph capture cannot wait for an event recorded
    // outside its graph: there the caller orders the calls (they are nodes of one graph, or the captures do not overlap).
    std::lock_guard<std::mutex> lock(g_attn_bwd_scratch_mu);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    EISEN_HIP_TRY(ctx, hipStreamIsCapturing(ctx->stream, &capture));
    hipEvent_t done = g_attn_bwd_scratch_done[ctx->device];
    const bool ordered = capture == hipStreamCaptureStatusNone && done != nullptr;
    if (ordered) EISEN_HIP_TRY(ctx, hipStreamWaitEvent(ctx->stream, done, 0));
    // per-kernel profiling creates events on first use: off for the duration of this call
    const bool prof_was = ctx->prof.enabled;
    ctx->prof.enabled = false;
    const int rc = attention_backward_common(ctx, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, q_strides, kv_strides, scale, causal,
                                             false, ctx->attn_scratch);
    ctx->prof.enabled = prof_was;
    if (ordered) EISEN_HIP_TRY(ctx, hipEventRecord(done, ctx->stream));
    return rc;
}

extern "C" int eisen_hip_attention_rope_backward(eisen_ctx* ctx, const void* q, const void* k, const void* v, const void* out,
                                                 const void* dout, const float* lse, void* dq, void* dk, void* dv, int dtype,
                                                 size_t B, size_t S, size_t Hq, size_t Hkv, size_t hd, float scale, int causal) {
    EISEN_CHECK_CTX(ctx);
    if (dtype == EISEN_BF16)  // the MFMA kernels rotate dQ and dK back as they store them
        return attention_backward_common(ctx, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, nullptr, nullptr, scale, causal, true);
    // f32 path: the plain backward, then the rotary backward in place
    int rc = attention_backward_common(ctx, q, k, v, out, dout, lse, dq, dk, dv, dtype, B, S, Hq, Hkv, hd, nullptr, nullptr, scale, causal, false);
    if (!rc) rc = eisen_hip_rope_backward(ctx, dq, dq, dtype, B, S, Hq * hd, hd, 0);
    if (!rc) rc = eisen_hip_rope_backward(ctx, dk, dk, dtype, B, S, Hkv * hd, hd, 0);
    return rc;
}
