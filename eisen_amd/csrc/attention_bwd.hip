// Flash-attention backward, the key-stationary pass: dK and dV (head_dim 32 and 64, bf16 MFMA).
//
//   dV = P^T dO,  dK = scale dS^T Q,  dS = P o (dO V^T - D),  P = exp2(log2e (scale Q K^T - LSE))
// summed over the query heads of a KV group (the repeat_kv backward, src/graph/ops/gqa.rs:168-184) and over every
// query that sees the key (the bmm backward of the reference's chain, src/graph/ops/linear.rs:1482-1498, and the
// softmax backward, src/graph/ops/reduction.rs:504-512).  The reference has no such kernel; what it must equal is
// that chain.
//
// Shape of the kernel
//   * A workgroup owns the keys of two 32-key blocks of one KV head, a heavy one and its light mirror image under the
//     causal mask (equal work everywhere).  Its four waves each take every fourth (query head of the group, 32-query
//     tile) item; their partial dK / dV meet in LDS once per key block, in wave order (no atomics).
//   * A tile is a chain of latencies per wave (loads issued, operand reads, two dependent MFMA groups with the softmax
//     between them) that the second wave of the SIMD covers in part.  So a wave must fit 256 registers (two per SIMD) and
//     should spend as few cycles as possible on anything but MFMAs and the softmax:
//       - every MFMA takes its accumulator in ordinary VGPRs (the file is compiled that way): with the AGPR form the
//         compiler copies the score accumulators between the register files around the softmax of every tile;
//       - Q / dO tiles and the two per-query statistics go from global memory straight into a private two-stage LDS
//         ring of the wave (global_load_lds with a scalar base: no staging registers, no LDS stores, no address
//         arithmetic in vector registers, no barrier in the loop);
//       - the score accumulator starts at -LSE / scale and the dP accumulator at D (read from the ring straight into
//         the accumulator registers), and the sign of V is flipped once per key block, so the MFMA chains deliver
//         S - LSE / scale and D - dP: a probability is one multiply and one exp2, -dS one more multiply; -scale is
//         applied when dK is stored.
#include "attention_common.cuh"

namespace {

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void mfma(f32x16& acc, const bf16x8& a, const bf16x8& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}

// ABL: a part of the tile loop left out for a measurement (AttnAblation; kAblNone is the kernel)
template <int HD, int ABL>
__global__ __launch_bounds__(256, 2) void fa_bwd_dkv32_kernel(AttnArgs a) {
    constexpr int KSTEPS = HD / 16, DT = HD / 32, NST = 2;
    constexpr int TILE = 32 * HD;                        // elements of a Q or dO tile
    constexpr int STAGE_BYTES = 2 * TILE * 2 + 256;      // Q tile, dO tile, 32 x (-LSE / scale | D)
    using Loader = DirectTile<HD, 32, 1>;
    constexpr int LOADS = 2 * Loader::PER_WAVE + 1;      // load instructions per tile
    static_assert(LOADS <= 63, "the tile in flight must fit the vmcnt counter");
    static_assert(2 * 4 * 32 * HD * sizeof(float) <= 4 * NST * STAGE_BYTES, "the reduction of dK and dV reuses the rings");
    __shared__ __attribute__((aligned(1024))) char lds[4 * NST * STAGE_BYTES];

    const int lane = threadIdx.x & 63, g = lane >> 5, c = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_qt = (a.S + 31) / 32, n_pairs = (n_qt + 1) / 2;
    // grid: x = key-block pair, fastest; then KV head, then batch.  Blocks of one (batch, KV head) read the same
    // Q / dO tiles, so they are kept on one XCD.
    const int bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int pair = bid % n_pairs, kvh = (bid / n_pairs) % a.Hkv, b = bid / (n_pairs * a.Hkv);
    char* ring = lds + wave * (NST * STAGE_BYTES);
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    // lanes 0-31 fetch the tile's -LSE / scale, lanes 32-63 its D: byte offset of the lane's value from D's entry for the
    // tile's first query (the launcher has checked that the statistics are less than 2 GiB apart)
    const unsigned stat_off = (unsigned)(g == 0 ? (a.L2 - a.D) * 4 : 0) + 4 * (unsigned)c;
    Loader loader;
    loader.init(a.q_ss, 0, lane);
    constexpr bool TL = ABL == kAblTimeline;
    attn_stamp<TL>(a, 2, kStampStart, lane, wave);

    // K and V rows of this lane's key of key block kb_, as they are stored
    bf16x8 kraw[KSTEPS], vraw[KSTEPS];
    auto load_kv = [&](int kb_) {
        const int key_ = kb_ * 32 + c;
        const long long koff = b * a.k_sb + kvh * a.k_sh + (long long)key_ * a.k_ss;
#pragma unroll
        for (int st = 0; st < KSTEPS; st++) {
            const int d = st * 16 + 8 * g;
            kraw[st] = key_ < a.S ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.K) + koff + d) : zero8;
            vraw[st] = key_ < a.S ? *reinterpret_cast<const bf16x8*>(static_cast<const bf16_t*>(a.V) + koff + d) : zero8;
        }
    };

    for (int pass = 0; pass < 2; pass++) {
        const int kb = pass == 0 ? pair : n_qt - 1 - pair;
        if (pass == 1 && kb <= pair) break;  // odd block count: the middle block has no mirror
        const int k0 = kb * 32;
        if (pass == 0) load_kv(kb);  // the second pass's rows were requested before the first pass's reduction
        f32x16 dk[DT], dv[DT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) { dk[dt][v] = 0.f; dv[dt][v] = 0.f; }

        const int qt_start = a.causal ? kb : 0;  // the diagonal tile is the first one that sees these keys
        const int per_head = n_qt - qt_start;
        const int n_items = a.G * per_head;       // (query head of the group, query tile), head-major
        const int n_mine = n_items > wave ? (n_items - wave + 3) / 4 : 0;

        auto stage_of = [&](int i) { return ring + (ABL == kAblTileLoads ? 0 : (i % NST)) * STAGE_BYTES; };
        // The tile that the next issue() requests, kept as running sums (all wave-uniform, so scalar registers): this wave's
        // items are wave, wave + 4, ... in head-major order; a step of four tiles that runs past the head's last tile
        // wraps into the next head.
        int nrel = wave % per_head;                    // tile index within the head, from the diagonal tile
        int nq0 = (qt_start + nrel) * 32;              // its first query
        long long ntile, nstat;                        // element offsets of its Q / dO rows and of its statistics
        {
            const int hq = kvh * a.G + wave / per_head;
            ntile = b * a.q_sb + hq * a.q_sh + (long long)nq0 * a.q_ss;
            nstat = ((long long)b * a.Hq + hq) * a.S + nq0;
        }
        const long long tile_wrap = a.q_sh - (long long)per_head * 32 * a.q_ss, stat_wrap = (long long)a.S - per_head * 32;
        auto issue = [&](int i) -> int {  // the loads of this wave's i-th tile into ring stage i % NST; returns the tile's first query
            const int q0 = nq0;
            char* stage = stage_of(i);
            const char* qbase = reinterpret_cast<const char*>(static_cast<const bf16_t*>(a.Q) + ntile);
            const char* dobase = reinterpret_cast<const char*>(static_cast<const bf16_t*>(a.dO) + ntile);
            const char* sbase = reinterpret_cast<const char*>(a.D + nstat);
            nrel += 4; nq0 += 128; ntile += 128 * a.q_ss; nstat += 128;
            while (nrel >= per_head) { nrel -= per_head; nq0 -= per_head * 32; ntile += tile_wrap; nstat += stat_wrap; }
            if (q0 + 32 <= a.S) {
#pragma unroll
                for (int r = 0; r < Loader::PER_WAVE; r++) {
                    load_lds_16(qbase, loader.off[r], stage + r * 1024);
                    load_lds_16(dobase, loader.off[r], stage + TILE * 2 + r * 1024);
                }
                load_lds_4(sbase, stat_off, stage + 2 * TILE * 2);
            } else {  // ragged last tile: rows past the end re-read the last row (they are given zero weight)
#pragma unroll
                for (int r = 0; r < Loader::PER_WAVE; r++) {
                    const int row = Loader::lane_row(0, r, lane), gr = min(row, a.S - 1 - q0);
                    const unsigned off = (unsigned)((gr * a.q_ss + Loader::lane_chunk(row, lane) * 8) * 2);
                    load_lds_16(qbase, off, stage + r * 1024);
                    load_lds_16(dobase, off, stage + TILE * 2 + r * 1024);
                }
                load_lds_4(sbase, stat_off - 4 * (unsigned)(c - min(c, a.S - 1 - q0)), stage + 2 * TILE * 2);
            }
            return q0;
        };

        int q0_next = n_mine > 0 ? issue(0) : 0;
        bf16x8 kf[KSTEPS], vn[KSTEPS];  // K and -V of the 32 keys, MFMA B operands (requested before the first tile, used after it is)
#pragma unroll
        for (int st = 0; st < KSTEPS; st++) {
            typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
            kf[st] = kraw[st];
            u32x4 bits = __builtin_bit_cast(u32x4, vraw[st]) ^ 0x80008000u;  // sign flip of the eight bf16 values
            vn[st] = __builtin_bit_cast(bf16x8, bits);
            // the flip is done here, once, not again at every use; and both operands have arrived before the loop (a
            // pending load of theirs would make the compiler wait for every outstanding load at their first use in it,
            // the prefetched tile's included)
            asm volatile("" : "+v"(vn[st]), "+v"(kf[st]));
        }
        attn_stamp<TL>(a, 2, kStampLoop + kStampsPerPass * pass, lane, wave);
        for (int i = 0; i < n_mine; i++) {
            wait_vmcnt<0>();  // tile i was requested in the middle of tile i - 1
            const int q0 = q0_next;
            const bf16_t* Qs = reinterpret_cast<const bf16_t*>(stage_of(i));
            const bf16_t* dOs = Qs + TILE;
            float* st = reinterpret_cast<float*>(stage_of(i) + 2 * TILE * 2);
            if (q0 + 32 > a.S) {  // a query past the end gets LSE = +inf (stored negated): its probabilities are exactly zero
                if (g == 0 && q0 + c >= a.S) st[c] = -INFINITY;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
            // scores: S - LSE / scale and D - dP, the start values read straight into the accumulator registers
            f32x16 s, dp;
#pragma unroll
            for (int vg = 0; vg < 4; vg++) {
                const float4 l4 = *reinterpret_cast<const float4*>(st + 8 * vg + 4 * g);
                const float4 d4 = *reinterpret_cast<const float4*>(st + 32 + 8 * vg + 4 * g);
                s[4 * vg] = l4.x; s[4 * vg + 1] = l4.y; s[4 * vg + 2] = l4.z; s[4 * vg + 3] = l4.w;
                dp[4 * vg] = d4.x; dp[4 * vg + 1] = d4.y; dp[4 * vg + 2] = d4.z; dp[4 * vg + 3] = d4.w;
            }
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ks++) {
                const bf16x8 qa = ABL == kAblOperandReads ? vn[ks] : *reinterpret_cast<const bf16x8*>(Qs + tile_at<HD>(c, ks * 16 + 8 * g));
                const bf16x8 da = ABL == kAblOperandReads ? kf[ks] : *reinterpret_cast<const bf16x8*>(dOs + tile_at<HD>(c, ks * 16 + 8 * g));
                if (ABL == kAblScoreMfmas) { s[ks] += (float)qa[0]; dp[ks] += (float)da[0]; }
                else {
                mfma(s, qa, kf[ks]);
                mfma(dp, da, vn[ks]);
                }
            }
            // the transposed operands of the accumulation, requested before the softmax so that they arrive under it
            bf16x8 dotr[DT][2], qtr[DT][2];
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    if (ABL == kAblTransposedReads) { dotr[dt][t] = kf[dt * 2 + t]; qtr[dt][t] = vn[dt * 2 + t]; }
                    else {
                    dotr[dt][t] = lds_tr_operand_swz<HD>(dOs, 0, dt * 32, t, lane);
                    qtr[dt][t] = lds_tr_operand_swz<HD>(Qs, 0, dt * 32, t, lane);
                    }
                }
            // the next tile's loads go out while the score MFMAs run (the other stage was read by tile i - 1, whose operand reads
            // have all returned)
            if (ABL != kAblTileLoads && i + 1 < n_mine) q0_next = issue(i + 1);
            float p[16];
#pragma unroll
            for (int v = 0; v < 16; v++) p[v] = ABL == kAblSoftmax ? s[v] : fast_exp2(s[v] * a.scale_log2e);
            // only the diagonal tile is cut by the causal mask
            if (a.causal && q0 == k0) {
                asm volatile("" ::: "memory");  // keeps this a branch taken once per head, not 16 selects per tile
#pragma unroll
                for (int v = 0; v < 16; v++)
                    if (c > acc_row(v, g)) p[v] = 0.f;  // key k0 + c is after query q0 + row
            }
            bf16x8 pf[2], dsf[2];
#pragma unroll
            for (int v = 0; v < 16; v++) {
                pf[v >> 3][v & 7] = (bf16_t)p[v];
                dsf[v >> 3][v & 7] = (bf16_t)(ABL == kAblSoftmax ? dp[v] : p[v] * dp[v]);  // = -dS: dp holds D - dP
            }
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    if (ABL == kAblSecondMfmas) { dv[dt][0] += (float)pf[t][0] * (float)dotr[dt][t][0]; dk[dt][0] += (float)dsf[t][0] * (float)qtr[dt][t][0]; }
                    else {
                    mfma(dv[dt], pf[t], dotr[dt][t]);
                    mfma(dk[dt], dsf[t], qtr[dt][t]);
                    }
                }
        }
        attn_stamp<TL>(a, 2, kStampLoopEnd + kStampsPerPass * pass, lane, wave);
        // the mirror block's K and V rows travel while this block's partial results are summed
        if (pass == 0 && n_qt - 1 - pair > pair) load_kv(n_qt - 1 - pair);
        // Sum the four waves' partial results through the (now idle) rings and store: dK and dV in one round.
        float* red = reinterpret_cast<float*>(lds);  // [dK | dV][wave][32 keys][HD]
        bf16_t* outs[2] = {static_cast<bf16_t*>(a.dK) + b * a.k_sb + kvh * a.k_sh, static_cast<bf16_t*>(a.dV) + b * a.k_sb + kvh * a.k_sh};
        __syncthreads();  // every wave is done with its ring
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int at = (wave * 32 + acc_row(v, g)) * HD + dt * 32 + c;
                red[at] = dk[dt][v] * -a.scale;
                red[4 * 32 * HD + at] = dv[dt][v];
            }
        __syncthreads();
#pragma unroll
        for (int which = 0; which < 2; which++) {
            for (int e0 = threadIdx.x * 8; e0 < 32 * HD; e0 += 256 * 8) {
                float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const float* src = red + (which * 4 + w) * 32 * HD + e0;
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
        __syncthreads();  // the reduction's reads are over before the next pass refills the rings
        attn_stamp<TL>(a, 2, kStampStored + kStampsPerPass * pass, lane, wave);
    }
}

}  // namespace

// What the kernel above covers: head_dim 32 and 64, and shapes whose byte offsets inside a tile (31 rows of the query
// stride) and between the two statistics arrays fit 32 bits.
bool eisen_attention_dkv32_supports(const AttnArgs& a) {
    return (a.hd == 32 || a.hd == 64) && a.q_ss > 0 && a.q_ss * 32 * 2 < (1ll << 31) && a.L2 > a.D && (a.L2 - a.D) * 4 < (1ll << 31);
}

// a.L2 (-LSE / scale) and a.D must have been written (by the dQ kernel).
void eisen_attention_launch_dkv32(eisen_ctx* ctx, const AttnArgs& a) {
    const int n_kb = (a.S + 31) / 32;  // 32-key blocks, handled in heavy / light pairs
    dim3 grid((unsigned)((n_kb + 1) / 2 * a.Hkv * a.B));
    if (a.hd == 64) {
        switch (a.ablation) {  // hd 64 only: the head size the measurements are quoted for
            case kAblTransposedReads: fa_bwd_dkv32_kernel<64, kAblTransposedReads><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblOperandReads: fa_bwd_dkv32_kernel<64, kAblOperandReads><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblSecondMfmas: fa_bwd_dkv32_kernel<64, kAblSecondMfmas><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblTileLoads: fa_bwd_dkv32_kernel<64, kAblTileLoads><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblSoftmax: fa_bwd_dkv32_kernel<64, kAblSoftmax><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblScoreMfmas: fa_bwd_dkv32_kernel<64, kAblScoreMfmas><<<grid, 256, 0, ctx->stream>>>(a); break;
            case kAblTimeline: fa_bwd_dkv32_kernel<64, kAblTimeline><<<grid, 256, 0, ctx->stream>>>(a); break;
            default: fa_bwd_dkv32_kernel<64, kAblNone><<<grid, 256, 0, ctx->stream>>>(a); break;
        }
    }
    else fa_bwd_dkv32_kernel<32, kAblNone><<<grid, 256, 0, ctx->stream>>>(a);
}
