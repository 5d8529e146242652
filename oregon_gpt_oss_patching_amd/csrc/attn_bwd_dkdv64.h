// dK / dV for long full-causal rows: one wavefront per SIMD, 64 keys per wavefront, the loop over (query
// tile, query head) software-pipelined by hand inside the wavefront.  Same arithmetic and the same order of
// additions per accumulator as attn_bwd_dkdv_kernel (the results have the same bits); what changes is
// how the work is issued.
//
// Why.  With 32 keys per wavefront (attn_bwd_dkdv_kernel) every Q / dO fragment read from LDS feeds ONE
// MFMA, which keeps the CU's LDS pipe as busy as its matrix pipes and leaves both half idle waiting for
// each other.  With 64 keys per wavefront a fragment feeds two MFMAs, but the accumulators (dK^T, dV^T:
// 64 x 64 floats each per wavefront = 128 registers) and the K / V fragments (64) then fill half of the
// 512-register file, so only one wavefront fits a SIMD and nobody else hides its latencies or shares the
// instruction issue: a lone wavefront issues one instruction every four cycles (eight for an MFMA or a
// transcendental), and 64 MFMAs of 32 cycles leave room for about 450 instructions per tile.  The overlap of
// matrix, vector and LDS work therefore has to be in the wavefront's own instruction order, across tile
// boundaries, and everything that is not arithmetic on the tile has to be nearly free:
//
//   a 64-row query tile against the wavefront's 64 keys = 4 substeps t = (32-row block qb = t / 2,
//   32-key block nb = t % 2), each
//     M1(t): S - lse / scale = Q K^T + (statistics step), dP - delta likewise      8 MFMAs + 2 for the statistics
//                                                                                   step of a row block, results in VGPRs
//     V(t):  P = exp2((S - lse / scale) c), dS = P (dP - delta), -> bf16           16 elements per lane
//     M2(t): dV^T += dO^T P, dK^T += Q^T dS                                        8 MFMAs, accumulators in AGPRs
//   issued as a steady stream of slots of 18 MFMAs: slot = { M2(t-1), M1(t+1), V(t), LDS reads }.
//   The streams of a slot are independent, so every MFMA is followed by one step of V and at most one
//   LDS read, and a scheduling fence pins that order.  The slot that starts a tile's last block also
//   holds the iteration's synchronisation (copy landed, barrier, next copy issued), so the tile
//   boundary costs no drain: M1 of the next tile's first substep is issued in the current tile's
//   last slot.
//
// The host sends only problems in which every wavefront meets, in walk order, at most one tile whose last
// rows are padding (masked), interior tiles, the query tile on its diagonal (masked), then tiles it has
// nothing to do with: bf16, full causal, Sq == Skv a multiple of 64, no offset, no packed rows; right-padded
// batch rows (seqlens) are fine.
#pragma once
#include "attn_bwd.h"

namespace gptoss {

struct Dkdv64 {
    static constexpr int NS = 3;       // LDS stages
    static constexpr int WK = 64;      // keys per wavefront
    static constexpr int BN = 256;     // keys per workgroup (4 wavefronts)
    static constexpr int kCopiesPerTile = 5;                       // vector-memory instructions one wavefront issues per staged tile
    static constexpr int kStatOff = 2 * kStageTileBytes;           // a stage: Q tile, dO tile, 64 rows of split statistics
    static constexpr int kStageBytes = kStatOff + kTile * 16;
    static constexpr int kWaveRows = 16;                           // rows of each tile one wavefront copies
};

template <bool PADDED>          // PADDED: right-padded batch rows (seqlens given)
__global__ __launch_bounds__(256, 1) void attn_bwd_dkdv64_kernel(const KArgs a) {
    using C = Dkdv64;
    constexpr int NS = C::NS, WK = C::WK, BN = C::BN, NB = 2;
    __shared__ __attribute__((aligned(16))) char smem[NS * C::kStageBytes];

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;

    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int b = bid % a.B; bid /= a.B;
    const int part = bid % a.dkdv_parts; bid /= a.dkdv_parts;
    const int kt = bid;                                   // ascending: most work first
    const int j0 = kt * BN;                               // first key of the workgroup
    const int wj0 = j0 + WK * w;                          // first key of the wavefront

    // The query tiles that can see the workgroup's keys run from the one that holds its first key to the
    // last one; with dkdv_parts > 1 they are cut into that many consecutive slices, one per workgroup, each
    // of which leaves an fp32 partial sum (attn_bwd_dkdv_reduce_kernel adds them in slice order).  The
    // workgroup walks its slice from the last tile down, all heads of the group per tile.  Wavefront w's
    // diagonal tile is tile wq; above it every tile is interior, below it none concerns the wavefront.
    // A right-padded batch row is a shorter row: rows and keys from len on do not exist.  Its last tile may be
    // partial (len not a multiple of 64): that one goes through the masked body before the interior tiles.
    const int len = PADDED ? max(0, min(a.Sq, a.seqlens[b])) : a.Sq;
    const int qt_all_hi = (len + kTile - 1) / kTile, qt_lo = j0 / kTile;
    const int nq_all = max(0, qt_all_hi - qt_lo);
    const int slice = (nq_all + a.dkdv_parts - 1) / a.dkdv_parts;
    const int qt_hi = qt_all_hi - part * slice;                       // end of this workgroup's slice
    const int nq = max(0, min(slice, nq_all - part * slice));
    const int n_it = nq * a.r;
    const int wq = qt_lo + w;                             // the query tile on the wavefront's diagonal
    const bool wave_live = wj0 < len;                     // (then wq < qt_all_hi)
    const int t_part = (len % kTile) ? qt_all_hi - 1 : -1;            // the partial tile, if there is one
    // in walk order: the partial tile if it is in this slice and above the diagonal, the interior tiles, the diagonal tile
    const bool top_here = PADDED && wave_live && t_part > wq && t_part == qt_hi - 1 && nq > 0;
    const int n_top = top_here ? a.r : 0;
    const int n_int = (wave_live ? max(0, min(nq, qt_hi - 1 - wq)) : 0) * a.r - n_top;
    const int n_mask = (wave_live && wq < qt_hi && wq >= qt_hi - nq) ? a.r : 0;

    // K, V fragments (B operands): lane = key, slots = head_dim
    bf16x8 kf[NB][4], vf[NB][4];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int j = wj0 + 32 * nb + l32;
        const bf16 *krow = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h + (int64_t)j * a.ks.s;
        const bf16 *vrow = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h + (int64_t)j * a.vs.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 zk = {0u, 0u, 0u, 0u}, zv = {0u, 0u, 0u, 0u};
            if (j < a.Skv) {
                zk = *reinterpret_cast<const u32x4 *>(krow + 16 * ks + 8 * half);
                zv = *reinterpret_cast<const u32x4 *>(vrow + 16 * ks + 8 * half);
            }
            kf[nb][ks] = as_bf16x8(zk);
            vf[nb][ks] = as_bf16x8(zv);
        }
    }
    f32x16 dk[NB][2], dv[NB][2];       // AGPRs: only mfma_bf16_agpr* touches them until the epilogue
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) { dk[nb][0][i] = dk[nb][1][i] = 0.0f; dv[nb][0][i] = dv[nb][1][i] = 0.0f; }

    const float c = a.scale_log2;
    bf16x8 b_stat_s, b_stat_dp;        // B operands of the statistics step
    stat_step_operands(half, b_stat_s, b_stat_dp);
    const uint32_t smem_base = lds_addr(&smem[0]);

    // ---- LDS addresses ----------------------------------------------------------------------------
    // Nine per-lane addresses into the stage being read (four natural fragments, four transposed ones, the
    // statistics row); the tile (Q / dO), the 32-row block and the 16-row step are immediates of the read.
    // They move from stage to stage by one add each per tile.
    uint32_t adr[9];
    {
        const TileLaneOffsets lo = make_tile_offsets(lane);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) adr[ks] = smem_base + lo.nat[ks];
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int t = 0; t < 2; ++t) adr[4 + 2 * dblk + t] = smem_base + lo.tr[dblk][t];
        adr[8] = smem_base + C::kStatOff + l32 * 16;
    }
    // Wave-uniform bases of the three stages in rotation (each already at the first row this wavefront copies):
    // c0 = the stage of the tile being consumed, which is also the one the next request fills once every
    // wavefront is done with it; c1 = the stage of the tile after it; c2 the third.
    uint32_t c0 = __builtin_amdgcn_readfirstlane(smem_base + w * (C::kWaveRows * kRowBytes));
    uint32_t c1 = c0 + C::kStageBytes, c2 = c1 + C::kStageBytes;
    auto rotate = [&]() __attribute__((always_inline)) { const uint32_t t = c0; c0 = c1; c1 = c2; c2 = t; };

    // ---- the copies: tiles are requested in walk order (query tiles from the last one down, heads inner) ----
    // Everything here is branch-free (selects only): the synchronisation sits in the middle of the pipelined
    // loop body, and a branch there would let the compiler sink vector work of earlier slots past it.  So
    // every wavefront issues exactly kCopiesPerTile copies per request (its 16 rows of Q and of dO as two
    // 1 KB pieces each, and its 16 rows of statistics as 64 dwords), and once the walk is exhausted a request
    // copies the last tile again into the stage that is free by then, so that "at most kCopiesPerTile
    // outstanding" keeps meaning "the tile before has landed".
    const AsyncLaneOffsets qlane = make_async_offsets(a.qs.s, lane, w), glane = make_async_offsets(a.dos.s, lane, w);
    const uint32_t stat_voff = w * (C::kWaveRows * 16) + lane * 4;
    const uint32_t stat_dst = __builtin_amdgcn_readfirstlane(C::kStatOff - w * (C::kWaveRows * kRowBytes) + w * (C::kWaveRows * 16));
    int iss_h = 0, iss_left = n_it;
    // The walk moves 32-bit byte offsets (the lanes' own, one vector add each per tile) over fixed bases: the
    // lowest tile of the slice, first head of the group.  Scalar instructions are the expensive ones for a
    // wavefront that has its SIMD to itself (about 8 cycles of issue each, a vector add 4), and 64-bit pointer
    // walks take many.  The host takes this kernel only when every such offset fits (dkdv64_route).
    const int n_tiles = a.Sq / kTile;
    const int t_base = max(0, min(qt_hi - nq, n_tiles - 1));          // (an empty slice requests tile t_base over and over)
    const int t_first = max(0, nq - 1);                                // tiles above t_base where the walk starts
    const bf16 *qbase = a.q + (int64_t)b * a.qs.b + (int64_t)(g * a.r) * a.qs.h + (int64_t)(t_base * kTile) * a.qs.s;
    const bf16 *gbase = a.d_o + (int64_t)b * a.dos.b + (int64_t)(g * a.r) * a.dos.h + (int64_t)(t_base * kTile) * a.dos.s;
    const u32x4 *stat_base = a.split + ((int64_t)b * a.H + (int64_t)g * a.r) * a.Sq + t_base * kTile;     // wave-uniform
    uint32_t qoff0 = qlane.off[0] + (uint32_t)(t_first * kTile) * (uint32_t)a.qs.s * 2u, qoff1 = qlane.off[1] + (uint32_t)(t_first * kTile) * (uint32_t)a.qs.s * 2u;
    uint32_t goff0 = glane.off[0] + (uint32_t)(t_first * kTile) * (uint32_t)a.dos.s * 2u, goff1 = glane.off[1] + (uint32_t)(t_first * kTile) * (uint32_t)a.dos.s * 2u;
    uint32_t soff = stat_voff + (uint32_t)(t_first * kTile) * 16u;
    // per request: on to the next head, or (after the last head of the group) back to the first head of the tile below
    const uint32_t q_step = (uint32_t)a.qs.h * 2u, q_wrap = 0u - ((uint32_t)(a.r - 1) * (uint32_t)a.qs.h + (uint32_t)kTile * (uint32_t)a.qs.s) * 2u;
    const uint32_t g_step = (uint32_t)a.dos.h * 2u, g_wrap = 0u - ((uint32_t)(a.r - 1) * (uint32_t)a.dos.h + (uint32_t)kTile * (uint32_t)a.dos.s) * 2u;
    const uint32_t s_step = (uint32_t)a.Sq * 16u, s_wrap = 0u - ((uint32_t)(a.r - 1) * (uint32_t)a.Sq + (uint32_t)kTile) * 16u;
    // copy `which` (0..4) of the current request into the stage at `dst`; advance() moves on to the next tile
    auto issue_one = [&](uint32_t dst, int which) __attribute__((always_inline)) {
        if (which == 0) lds_dma16_plus<0>(dst, qbase, qoff0);
        if (which == 1) lds_dma16_plus<8 * kRowBytes>(dst, qbase, qoff1);
        if (which == 2) lds_dma16_plus<kStageTileBytes>(dst, gbase, goff0);
        if (which == 3) lds_dma16_plus<kStageTileBytes + 8 * kRowBytes>(dst, gbase, goff1);
        if (which == 4) lds_dma4_at(dst, stat_dst, stat_base, soff);
    };
    auto advance = [&]() __attribute__((always_inline)) {
        const bool more = iss_left > 1;                 // another tile to request after this one
        const bool wrap = iss_h + 1 == a.r;
        const uint32_t dq_ = more ? (wrap ? q_wrap : q_step) : 0u;
        const uint32_t dg_ = more ? (wrap ? g_wrap : g_step) : 0u;
        const uint32_t ds_ = more ? (wrap ? s_wrap : s_step) : 0u;
        qoff0 += dq_; qoff1 += dq_;
        goff0 += dg_; goff1 += dg_;
        soff += ds_;
        iss_h = wrap ? 0 : iss_h + 1;
        iss_left -= 1;
    };
    auto issue = [&](uint32_t dst) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::kCopiesPerTile; ++i) issue_one(dst, i);
        advance();
    };
    // arrive(): the tile to be read next has landed in every wavefront and every wavefront is done reading
    // the tile before it, whose stage the request that follows then overwrites.  Every wavefront calls
    // arrive() + a request exactly n_it + 1 times, from wherever it is in its own instruction stream.
    auto arrive = [&]() __attribute__((always_inline)) {
        wait_vmcnt<C::kCopiesPerTile>();
        __syncthreads();
    };

    // ---- pipeline state (lives across tiles) ------------------------------------------------------------
    bf16x8 aq[2][4], ag[2][4];            // [qb][ks]   natural fragments of Q and dO
    bf16x8 aqt[2][2][2], agt[2][2][2];    // [qb][u][dblk] transposed fragments
    bf16x8 ast[2];                        // [qb]       split statistics of row l32 (A operand of the statistics step)
    f32x16 s[4], dp[4];
    bf16x8 pf[4][2], dsf[4][2];
#define GPTOSS_FENCE() __builtin_amdgcn_sched_barrier(0)

    // LDS reads of 32-row block qb of the stage the addresses point at, in units: 0..7 natural fragments (one
    // read each, Q for ks = 0..3 then dO), 8 the row statistics (one read), 16..23 transposed fragments (two
    // reads each)
    auto rd = [&](int qb, int unit) __attribute__((always_inline)) {
        if (unit < 8) {
            const int ks = unit & 3;
            const bf16x8 f = as_bf16x8(lds_load128(adr[ks], (unit >= 4 ? kStageTileBytes : 0) + 32 * qb * kRowBytes));
            if (unit >= 4) ag[qb][ks] = f; else aq[qb][ks] = f;
        } else if (unit == 8) {
            ast[qb] = as_bf16x8(lds_load128(adr[8], 32 * qb * 16));
        } else {
            const int j = unit - 16, u = j >> 2, dblk = (j >> 1) & 1;
            const int imm = ((j & 1) ? 0 : kStageTileBytes) + (32 * qb + 16 * u) * kRowBytes;
            union { struct { s16x4 a, b; } s; bf16x8 v; } x;
            x.s.a = lds_load_tr64(adr[4 + 2 * dblk], imm);
            x.s.b = lds_load_tr64(adr[5 + 2 * dblk], imm);
            if (j & 1) aqt[qb][u][dblk] = x.v; else agt[qb][u][dblk] = x.v;
        }
    };
    // MFMA j (0..9) of M1(t): S first (its exponentials are what the next slot starts with), each chain led by
    // its statistics step; MFMA j (0..7) of M2(t)
    // (The statistics step does not depend on the key block: it is issued once per 32-row block, with the first
    // key block, and both key blocks' chains start from its result.)
    f32x16 s_init[2], dp_init[2];
    auto m1 = [&](int t, int j) __attribute__((always_inline)) {
        const int qb = t >> 1, nb = t & 1;
        if (j == 0 || j == 5) {
            if (nb == 0) {
                f32x16 z;
#pragma unroll
                for (int i = 0; i < 16; ++i) z[i] = 0.0f;
                if (j == 0) s_init[qb] = mfma_bf16(ast[qb], b_stat_s, z); else dp_init[qb] = mfma_bf16(ast[qb], b_stat_dp, z);
            }
        } else if (j < 5) {
            s[t] = mfma_bf16(aq[qb][j - 1], kf[nb][j - 1], j == 1 ? s_init[qb] : s[t]);
        } else {
            dp[t] = mfma_bf16(ag[qb][j - 6], vf[nb][j - 6], j == 6 ? dp_init[qb] : dp[t]);
        }
    };
    // (t = 3 is the substep whose M2 follows a join of control flow: the top of the loop body and the drain;
    // a copy of an accumulator that the compiler places there may sit right in front of it)
    auto m2 = [&](int t, int j) __attribute__((always_inline)) {
        const int qb = t >> 1, nb = t & 1, u = j >> 2, dblk = (j >> 1) & 1;
        if (t == 3 && j < 4) {
            if (j & 1) mfma_bf16_agpr<true>(dk[nb][dblk], aqt[qb][u][dblk], dsf[t][u]);
            else mfma_bf16_agpr<true>(dv[nb][dblk], agt[qb][u][dblk], pf[t][u]);
        } else {
            if (j & 1) mfma_bf16_agpr<false>(dk[nb][dblk], aqt[qb][u][dblk], dsf[t][u]);
            else mfma_bf16_agpr<false>(dv[nb][dblk], agt[qb][u][dblk], pf[t][u]);
        }
    };
    // Step i (0..17) of V(t), three elements in flight so that no instruction of a step depends on
    // another one of the same step: the scaled logit of element i (S arrives with lse / scale already
    // taken off), the exponential of element i - 1, the product of element i - 2 and the packing of the
    // pair it completes.
    // MASKED (the diagonal tile, a partial last tile): pair (row r of the tile, the lane's key j of block nb) is
    // visible iff 0 <= dbase + r and r < row_lim, with dbase = (first position of the tile) - j, or hugely
    // negative for a key that does not exist; folded per lane and tile into (unsigned)(mdb[nb] + rc) < mwd[nb]
    // with rc the compile-time part of the row index (one add, one compare, one select per element, on the
    // logit: an invisible pair gets -inf and so P = dS = 0).
    // (Without padded rows only the diagonal tile is masked, every key exists and every row too: the two numbers
    // are constants of the lane, set here once.)
    int mdb[NB];
    unsigned mwd[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        mdb[nb] = 4 * half - (32 * nb + l32);
        mwd[nb] = (unsigned)(kTile - (32 * nb + l32));
    }
    auto set_mask = [&](int tile) __attribute__((always_inline)) {
        const int pos0 = tile * kTile, row_lim = min(kTile, len - pos0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int j = wj0 + 32 * nb + l32;
            const int dbase = j < len ? pos0 - j : -0x40000000;
            mdb[nb] = dbase + 4 * half;
            mwd[nb] = (unsigned)max(0, mdb[nb] + row_lim - 4 * half);
        }
    };
    auto vstep = [&](auto masked_, int t, int i) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_)::value;
        const int qb = t >> 1, nb = t & 1;
        if (i < 16) {
            float x = s[t][i] * c;
            if constexpr (MASKED) x = (unsigned)(mdb[nb] + (32 * qb + 8 * (i >> 2) + (i & 3))) < mwd[nb] ? x : -INFINITY;
            s[t][i] = x;
        }
        if (i >= 1 && i <= 16) s[t][i - 1] = fast_exp2(s[t][i - 1]);
        if (i >= 2) {
            const int k = i - 2;
            dp[t][k] = s[t][k] * dp[t][k];
            if (k & 1) {
                const int u = k >> 3, e = k & 7;
                pf[t][u][e - 1] = (bf16)s[t][k - 1];
                pf[t][u][e] = (bf16)s[t][k];
                dsf[t][u][e - 1] = (bf16)dp[t][k - 1];
                dsf[t][u][e] = (bf16)dp[t][k];
            }
        }
    };
    // One slot of 18 MFMAs.  MFMAs 0..7: M2(TP) (its packed operands were finished by the slot before; the
    // inline-assembly MFMAs therefore never end a slot, see mfma_bf16_agpr).  MFMAs 8..17: M1(TN).  Every
    // MFMA is followed by one step of V(TC) and by the LDS reads of block RQB: RKIND 1 = the row statistics
    // first and the natural fragments behind the MFMAs of M1 (each right after the MFMA that used the
    // fragment of the other block last, so the registers can be the same), RKIND 2 = transposed fragments.
    // SYNC: the iteration's synchronisation, the move of the read addresses to the next stage and the next
    // request (into the stage of the tile this iteration finishes), dealt out over the first micro-slots.
    auto slot = [&](auto masked_, auto tn_, auto tp_, auto tc_, auto rkind_, auto rqb_, auto sync_) __attribute__((always_inline)) {
        constexpr int TN = decltype(tn_)::value, TP = decltype(tp_)::value, TC = decltype(tc_)::value;
        constexpr int RKIND = decltype(rkind_)::value, RQB = decltype(rqb_)::value;
        constexpr bool SYNC = decltype(sync_)::value;
        if constexpr (SYNC) {
            arrive();
            GPTOSS_FENCE();
            const uint32_t step = c1 - c0;
#pragma unroll
            for (int i = 0; i < 9; ++i) adr[i] += step;
        }
#pragma unroll
        for (int m = 0; m < 18; ++m) {
            if (m < 8) m2(TP, m); else m1(TN, m - 8);
            vstep(masked_, TC, m);
            // M1 MFMA j = m - 8 uses natural fragment j - 1 (j = 1..4) or j - 2 (j = 6..9)
            if (RKIND == 1 && m == 0) rd(RQB, 8);
            if (RKIND == 1 && m >= 9 && m != 13) rd(RQB, m < 13 ? m - 9 : m - 10);
            if (RKIND == 2 && (m & 1) == 0 && m < 16) rd(RQB, 16 + (m >> 1));
            if constexpr (SYNC) {
                if (m >= 2 && m < 2 + C::kCopiesPerTile) issue_one(c0, m - 2);
                if (m == 2 + C::kCopiesPerTile) advance();
            }
            GPTOSS_FENCE();
        }
    };
    using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
    using T = std::true_type; using F = std::false_type;

    issue(c0);
    issue(c1);
    // The compiler does not see the copies (lds_dma16), but it does see this wait: from here on it knows
    // that the K / V loads above have arrived and puts no vmcnt wait of its own into the loops, where such
    // a wait would also drain the copies in flight.
    wait_vmcnt<0>();
    arrive();
    issue(c2);

    // one tile through the four slots
    auto body = [&](auto masked_) __attribute__((always_inline)) {
        GPTOSS_FENCE();
        // slot A: M2(3 of the tile before), M1(1) | V(0) | block 1: statistics, natural fragments
        slot(masked_, I1{}, I3{}, I0{}, I1{}, I1{}, F{});
        // slot B: M2(0), M1(2) | V(1) | block 1: transposed fragments
        slot(masked_, I2{}, I0{}, I1{}, I2{}, I1{}, F{});
        // slot C: the next tile has landed (and this one's stage is free for the request after next);
        //         M2(1), M1(3) | V(2) | next tile, block 0: statistics, natural fragments
        // slot D: M2(2), M1(0 of the next tile) | V(3) | next tile, block 0: transposed fragments
        // (When the run ends here the next tile's part is still issued, on whatever the next stage holds:
        // staged data of a tile this wavefront skips, or a repeated copy after the last tile.  Its results
        // are never used; the body stays free of variants and branches.)
        slot(masked_, I3{}, I1{}, I2{}, I1{}, I0{}, T{});
        slot(masked_, I0{}, I2{}, I3{}, I2{}, I0{}, F{});
        rotate();
    };

    if (n_top + n_int + n_mask > 0) {
        {   // fill: block 0 of the first tile, M1(0).  The first slot of the loop also issues M2 of "the tile
            // before": for the first tile that is a product of zeros (exact: the accumulators keep their
            // bits), which keeps the loop body free of variants.
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pf[3][u][e] = (bf16)0.0f;
                    dsf[3][u][e] = (bf16)0.0f;
#pragma unroll
                    for (int dblk = 0; dblk < 2; ++dblk) { aqt[1][u][dblk][e] = (bf16)0.0f; agt[1][u][dblk][e] = (bf16)0.0f; }
                }
            GPTOSS_FENCE();
#pragma unroll
            for (int unit = 0; unit < 9; ++unit) rd(0, unit);
            GPTOSS_FENCE();
#pragma unroll
            for (int j = 0; j < 10; ++j) {
                m1(0, j);
                if (j < 8) rd(0, 16 + j);
                GPTOSS_FENCE();
            }
        }
        // Interior tiles, then the diagonal tile: two plain counted loops one after the other rather than one
        // loop with two bodies, which the register allocator cannot hold together.  The pipeline state passes
        // from the first to the second.
        // (The explicit waits in front of the loops: whatever loads the compiler itself has in flight here,
        // reloads of spilled registers included, are then known to have arrived, and it puts no vmcnt wait of
        // its own into the loops, where it would drain the copies in flight on every pass.)
        if constexpr (PADDED) {
            // two phases of the same two loops, masked then interior: the partial tile and the interior tiles,
            // then the diagonal tile and nothing
#pragma unroll 1
            for (int ph = 0; ph < 2; ++ph) {
                const int nm = ph == 0 ? n_top : n_mask, ni = ph == 0 ? n_int : 0;
                set_mask(ph == 0 ? t_part : wq);
                wait_vmcnt<0>();
                for (int it = 0; it < nm; ++it) body(T{});
                wait_vmcnt<0>();
                for (int it = 0; it < ni; ++it) body(F{});
            }
        } else {
            wait_vmcnt<0>();
            for (int it = 0; it < n_int; ++it) body(F{});
            wait_vmcnt<0>();
            for (int it = 0; it < n_mask; ++it) body(T{});
        }
        // drain: M2(3)
        GPTOSS_FENCE();
#pragma unroll
        for (int j = 0; j < 8; ++j) m2(3, j);
        agpr_accumulators_settled(dk, dv);
    }
    // ---- the rest of the walk: nothing to compute, but every wavefront keeps the workgroup's rhythm of
    // barriers and requests ----
    for (int k = n_top + n_int + n_mask; k < n_it; ++k) {
        arrive();
        issue(c0);
        rotate();
    }
#undef GPTOSS_FENCE

    wait_vmcnt<0>();          // the repeated copies of the last requests
    agpr_accumulators_settled(dk, dv);
    if (a.dkdv_parts > 1) {
        // unscaled fp32 partial sums; lane = key row, register i of block dblk = column 32*dblk + crow(i, half),
        // four consecutive columns per 16-byte store
        const int64_t tensor = (int64_t)a.B * a.G * a.Skv * kD;
        float *pk = a.dkdv_partial + (int64_t)part * 2 * tensor + (((int64_t)b * a.G + g) * a.Skv) * kD;
        float *pv = pk + tensor;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int j = wj0 + 32 * nb + l32;
            if (j < a.Skv) {
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
                    for (int a4 = 0; a4 < 4; ++a4) {
                        const int col = 32 * dblk + 8 * a4 + 4 * half;
                        f32x4 xk, xv;
#pragma unroll
                        for (int e = 0; e < 4; ++e) { xk[e] = dk[nb][dblk][4 * a4 + e]; xv[e] = dv[nb][dblk][4 * a4 + e]; }
                        *reinterpret_cast<f32x4 *>(pk + (int64_t)j * kD + col) = xk;
                        *reinterpret_cast<f32x4 *>(pv + (int64_t)j * kD + col) = xv;
                    }
            }
        }
        return;
    }
    __syncthreads();
    bf16 *stage_out = reinterpret_cast<bf16 *>(&smem[0]) + w * 32 * kLS;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int r0 = wj0 + 32 * nb;
        const int nvalid = a.Skv - r0;
        store_rows32(stage_out, dk[nb], a.scale, a.dk + (int64_t)b * a.dks.b + (int64_t)g * a.dks.h + (int64_t)r0 * a.dks.s,
                     a.dks.s, nvalid, lane);
        __builtin_amdgcn_wave_barrier();
        store_rows32(stage_out, dv[nb], 1.0f, a.dv + (int64_t)b * a.dvs.b + (int64_t)g * a.dvs.h + (int64_t)r0 * a.dvs.s,
                     a.dvs.s, nvalid, lane);
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace gptoss
