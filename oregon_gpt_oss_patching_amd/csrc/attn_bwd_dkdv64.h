// dK / dV for long rows: one wavefront per SIMD, 64 keys per wavefront, the loop over (query tile,
// query head) software-pipelined by hand inside the wavefront.  Same arithmetic and the same order of
// additions per accumulator as attn_bwd_dkdv_kernel (the results have the same bits); what changes is
// how the work is issued.
//
// Why.  With 32 keys per wavefront (attn_bwd_dkdv_kernel) every Q / dO fragment read from LDS feeds ONE
// MFMA: 64 LDS instructions per 32 MFMAs, which keeps the CU's LDS pipe as busy as its matrix pipes and
// leaves both half idle waiting for each other.  With 64 keys per wavefront a fragment feeds two MFMAs,
// but the accumulators (dK^T, dV^T: 64 x 64 floats each per wavefront = 128 registers) and the K / V
// fragments (64) then fill half of the 512-register file, so only one wavefront fits a SIMD and nobody
// else hides its latencies.  The overlap of matrix, vector and LDS work therefore has to be in the
// wavefront's own instruction order, across tile boundaries:
//
//   a 64-row query tile against the wavefront's 64 keys = 4 substeps t = (32-row block qb = t / 2,
//   32-key block nb = t % 2), each
//     M1(t): S = Q K^T, dP = dO V^T - delta           8 MFMAs, results in VGPRs
//     V(t):  P = exp2(S c - lse2), dS = P dP, -> bf16  16 elements per lane
//     M2(t): dV^T += dO^T P, dK^T += Q^T dS            8 MFMAs, accumulators in AGPRs
//   issued as a steady stream of slots of 16 MFMAs: slot(t) = { M1(t+1), M2(t-1), V(t), 16 LDS reads }.
//   The three streams of a slot are independent, so every MFMA is followed by one element of V and one
//   LDS read, and a scheduling fence pins that order.  The slot that starts a tile's last block also
//   holds the iteration's synchronisation (copy landed, barrier, next copy issued), so the tile
//   boundary costs no drain: M1 of the next tile's first substep is issued in the current tile's
//   last slot.
//
// Tiles that need masking (the diagonal of a causal layer, window edges, padded rows) are rare on long
// rows; they leave the pipeline (it drains) and run dkdv_tile<true, ...> on the same accumulators.
#pragma once
#include "attn_bwd.h"

namespace gptoss {

struct Dkdv64 {
    static constexpr int NS = 3;       // LDS stages
    static constexpr int WK = 64;      // keys per wavefront
    static constexpr int BN = 256;     // keys per workgroup (4 wavefronts)
    static constexpr int kCopiesPerTile = 5;   // vector-memory instructions one wavefront issues per staged tile
};

__global__ __launch_bounds__(256, 1) void attn_bwd_dkdv64_kernel(const KArgs a) {
    using C = Dkdv64;
    constexpr int NS = C::NS, WK = C::WK, BN = C::BN, NB = 2;
    const int q_offset = query_offset(a);
    __shared__ __attribute__((aligned(16))) char smem[NS][2][kStageTileBytes];
    __shared__ __attribute__((aligned(16))) float sstat[NS][2][kTile];

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;

    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int b = bid % a.B; bid /= a.B;
    const int part = bid % a.dkdv_parts; bid /= a.dkdv_parts;
    const int kt = bid;                                   // ascending: most work first
    const int j0 = kt * BN;                               // first key of the workgroup
    const int wj0 = j0 + WK * w;                          // first key of the wavefront

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window ? a.window : 0x3fffffff;

    // query tiles that can see any key of the workgroup; with dkdv_parts > 1 this workgroup takes one
    // slice of them (as in attn_bwd_dkdv_kernel)
    const int j1 = min(j0 + BN, kv_len) - 1;
    const int i_lo = max(0, j0 - q_offset);
    int64_t i_hi64 = min((int64_t)a.Sq, (int64_t)q_len - q_offset);
    i_hi64 = min(i_hi64, (int64_t)j1 + weff - q_offset);
    const int i_hi = (j1 >= j0) ? (int)max((int64_t)0, i_hi64) : 0;
    const int qt_lo = i_lo / kTile;
    const int qt_all_hi = (i_hi + kTile - 1) / kTile;
    const int nq_all = max(0, qt_all_hi - qt_lo);
    const int slice = (nq_all + a.dkdv_parts - 1) / a.dkdv_parts;
    const int qt_hi = qt_all_hi - part * slice;
    const int nq = max(0, min(slice, nq_all - part * slice));
    const int n_it = nq * a.r;

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
    const float *lse2 = a.delta + (int64_t)a.B * a.H * a.Sq;
    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(&smem[0][0][0]), stat_base = lds_addr(&sstat[0][0][0]);
    int jkey[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) jkey[nb] = wj0 + 32 * nb + l32;

    // ---- the copies: tiles are requested in walk order (query tiles from the last one down, heads inner) ----
    // Everything here is branch-free (selects only): the synchronisation sits in the middle of the pipelined
    // loop body, and a branch there would let the compiler sink vector work of earlier slots past it.  So
    // every wavefront issues exactly kCopiesPerTile copies per request (the row statistics are copied by
    // wavefronts 0 and 1 and, to the same place, again by 2 and 3), the host guarantees Sq % 64 == 0 (no
    // clamped rows), and once the walk is exhausted a request copies the last tile again into the stage that
    // is free by then, so that "at most kCopiesPerTile outstanding" keeps meaning "the tile before has landed".
    const AsyncLaneOffsets qlane = make_async_offsets(a.qs.s, lane, w), glane = make_async_offsets(a.dos.s, lane, w);
    int iss_h = 0, iss_stage = 0, iss_left = n_it;
    const int i0_first = (qt_hi - 1) * kTile;
    const bf16 *qtile = a.q + (int64_t)b * a.qs.b + (int64_t)(g * a.r) * a.qs.h + (int64_t)i0_first * a.qs.s;
    const bf16 *gtile = a.d_o + (int64_t)b * a.dos.b + (int64_t)(g * a.r) * a.dos.h + (int64_t)i0_first * a.dos.s;
    // row statistics as staged: per 32-row block, 32 values of lse * log2(e) then its 32 values of -delta;
    // lanes 0..31 of a wavefront copy the former, lanes 32..63 the latter, for block w % 2
    const float *stat_src = (half ? a.delta : lse2) + ((int64_t)b * a.H + (int64_t)g * a.r) * a.Sq + i0_first + 32 * (w & 1) + l32;
    const int64_t q_step = a.qs.h, q_wrap = a.qs.h - (int64_t)a.r * a.qs.h - (int64_t)kTile * a.qs.s;
    const int64_t g_step = a.dos.h, g_wrap = a.dos.h - (int64_t)a.r * a.dos.h - (int64_t)kTile * a.dos.s;
    const int64_t s_step = a.Sq, s_wrap = (int64_t)a.Sq - (int64_t)a.r * a.Sq - kTile;
    // wave-uniform LDS destinations of stage 0 (the asynchronous copy takes its LDS base from M0)
    const uint32_t dst_tile = __builtin_amdgcn_readfirstlane(smem_base + w * (16 * kRowBytes));
    const uint32_t dst_stat = __builtin_amdgcn_readfirstlane(stat_base + (w & 1) * 256);
    // copy `which` (0..4) of the current request; advance() moves on to the next tile
    auto issue_one = [&](int which) __attribute__((always_inline)) {
        const uint32_t dt = dst_tile + iss_stage * (2 * kStageTileBytes);
        if (which == 0) lds_dma16(dt, qtile, qlane.off[0]);
        if (which == 1) lds_dma16(dt + 8 * kRowBytes, qtile, qlane.off[1]);
        if (which == 2) lds_dma16(dt + kStageTileBytes, gtile, glane.off[0]);
        if (which == 3) lds_dma16(dt + kStageTileBytes + 8 * kRowBytes, gtile, glane.off[1]);
        if (which == 4) lds_dma4_at(dst_stat + iss_stage * (2 * kTile * 4), stat_src);
    };
    auto advance = [&]() __attribute__((always_inline)) {
        const bool more = iss_left > 1;                 // another tile to request after this one
        const bool wrap = iss_h + 1 == a.r;
        qtile += more ? (wrap ? q_wrap : q_step) : 0;
        gtile += more ? (wrap ? g_wrap : g_step) : 0;
        stat_src += more ? (wrap ? s_wrap : s_step) : 0;
        iss_h = wrap ? 0 : iss_h + 1;
        iss_left = max(iss_left - 1, 0);
        iss_stage = iss_stage == NS - 1 ? 0 : iss_stage + 1;
    };
    auto issue = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < C::kCopiesPerTile; ++i) issue_one(i);
        advance();
    };
    // arrive(): the tile to be read next has landed in every wavefront and every wavefront is done reading
    // the tile before it, whose stage the request that follows then overwrites.  Every wavefront calls
    // arrive() + a request exactly n_it + 1 times, from wherever it is in its own instruction stream.
    auto arrive = [&]() __attribute__((always_inline)) {
        wait_vmcnt<C::kCopiesPerTile>();
        __syncthreads();
    };

    // ---- the tile being consumed -------------------------------------------------------------------
    int cur_h = 0, cur_i0 = i0_first, cur_stage = 0;
    enum { kSkip = 0, kInterior = 1, kMasked = 2 };
    // class of a query tile for this wavefront (the same for every head of the group)
    auto classify = [&](int i0) __attribute__((always_inline)) -> int {
        const int pos0 = q_offset + i0;
        const int pos1 = min(q_offset + min(a.Sq, i0 + kTile) - 1, q_len - 1);
        const int wj1 = min(wj0 + WK, kv_len) - 1;
        const bool skip = wj1 < wj0 || pos1 < wj0 || pos0 > wj1 + weff - 1 || pos1 < pos0;
        const bool interior = (wj0 + WK - 1 <= pos0) && (wj0 > pos1 - weff) && (wj0 + WK <= kv_len) &&
                              (q_offset + i0 + kTile - 1 <= pos1);
        return skip ? kSkip : (interior ? kInterior : kMasked);
    };

    // ---- pipeline state (lives across tiles) ------------------------------------------------------------
    bf16x8 aq[2][4], ag[2][4];            // [qb][ks]   natural fragments of Q and dO
    bf16x8 aqt[2][2][2], agt[2][2][2];    // [qb][u][dblk] transposed fragments
    f32x4 lv[2][4], nd[2][4];             // [qb][a4]   lse * log2(e), -delta of the accumulator rows
    f32x16 s[4], dp[4];
    bf16x8 pf[4][2], dsf[4][2];
#define GPTOSS_FENCE() __builtin_amdgcn_sched_barrier(0)

    // LDS reads of 32-row block qb of the tile staged at `st` (its row statistics at `stl`), in 24 units:
    // 0..7 natural fragments (one read each), 8..15 row statistics (one read each), 16..23 transposed
    // fragments (two reads each)
    auto rd = [&](uint32_t st, uint32_t stl, int qb, int unit) __attribute__((always_inline)) {
        const uint32_t qsm = st, gsm = st + kStageTileBytes;
        if (unit < 8) {
            const int ks = unit >> 1;
            if (unit & 1) ag[qb][ks] = ofrag_nat(gsm, lo, qb, ks); else aq[qb][ks] = ofrag_nat(qsm, lo, qb, ks);
        } else if (unit < 16) {
            const int a4 = (unit - 8) >> 1;
            if (unit & 1) lv[qb][a4] = lds_load128f(stl, (64 * qb + 8 * a4) * 4);
            else nd[qb][a4] = lds_load128f(stl, (64 * qb + 32 + 8 * a4) * 4);
        } else {
            const int j = unit - 16, u = j >> 2, dblk = (j >> 1) & 1;
            if (j & 1) aqt[qb][u][dblk] = ofrag_tr(qsm, lo, qb, u, dblk); else agt[qb][u][dblk] = ofrag_tr(gsm, lo, qb, u, dblk);
        }
    };
    // MFMA j (0..7) of M1(t) / M2(t)
    auto m1 = [&](int t, int j) __attribute__((always_inline)) {
        const int qb = t >> 1, nb = t & 1, ks = j >> 1;
        if (j == 0) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[t][i] = 0.0f;
        }
        if (j == 1) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4)
#pragma unroll
                for (int e = 0; e < 4; ++e) dp[t][4 * a4 + e] = nd[qb][a4][e];
        }
        if (j & 1) dp[t] = mfma_bf16(ag[qb][ks], vf[nb][ks], dp[t]); else s[t] = mfma_bf16(aq[qb][ks], kf[nb][ks], s[t]);
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
    // another one of the same step: the scaled logit of element i, the exponential of element i - 1,
    // the product of element i - 2 and the packing of the pair it completes.
    // MASKED: pair (row r of the tile, the lane's key of block nb) is visible iff 0 <= dbase + r < weff and
    // r < row_lim, folded per lane and tile into (unsigned)(mdb[nb] + rc) < mwd[nb] with rc the compile-time
    // part of the row index (one add, one compare, one select per element, on the logit: an invisible pair
    // gets -inf and so P = dS = 0, and steps 16 and 17, which finish a substep in the slot after its own,
    // need no mask).
    int mdb[NB] = {0, 0};
    unsigned mwd[NB] = {0u, 0u};
    auto vstep = [&](auto masked_, int t, int i) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_)::value;
        const int qb = t >> 1, nb = t & 1;
        if (i < 16) {
            float x = fmaf(s[t][i], c, -lv[qb][i >> 2][i & 3]);
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
    // One slot of 16 MFMAs.  MFMAs 0..7: M2(TP) (its packed operands were finished by the slot before and
    // by the two tail steps at the top of this one; the inline-assembly MFMAs therefore never end a slot,
    // see mfma_bf16_agpr).  MFMAs 8..15: M1(TN).  Every MFMA is followed by one step of V(TC) and by the
    // LDS reads of block RQB of the tile staged at (st, stl): RKIND 1 = row statistics behind MFMAs 0..7
    // and the natural fragments behind MFMAs 8..15 (each right after the MFMA that used the fragment of
    // the other block last, so the registers can be the same), RKIND 2 = transposed fragments.
    // SYNC: the iteration's synchronisation and the next request, dealt out over the first micro-slots.
    auto slot = [&](auto masked_, auto tn_, auto tp_, auto tc_, auto rkind_, auto rqb_, auto sync_, uint32_t st, uint32_t stl) __attribute__((always_inline)) {
        constexpr int TN = decltype(tn_)::value, TP = decltype(tp_)::value, TC = decltype(tc_)::value;
        constexpr int RKIND = decltype(rkind_)::value, RQB = decltype(rqb_)::value;
        constexpr bool SYNC = decltype(sync_)::value;
        constexpr int TV = (TC + 3) & 3;     // the substep whose last two steps are finished here
#ifndef GPTOSS_ABL_NOSYNC
        if constexpr (SYNC) { arrive(); GPTOSS_FENCE(); }
#endif
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            if (m < 8) m2(TP, m); else m1(TN, m - 8);
#ifndef GPTOSS_ABL_NOV
            if (m < 2) vstep(std::false_type{}, TV, 16 + m);
            vstep(masked_, TC, m);
#endif
#ifndef GPTOSS_ABL_NOLDS
            if (RKIND == 1) rd(st, stl, RQB, (m + 8) & 15);
            if (RKIND == 2 && (m & 1) == 0) rd(st, stl, RQB, 16 + (m >> 1));
#endif
#ifndef GPTOSS_ABL_NODMA
            if constexpr (SYNC) {
                if (m >= 2 && m < 2 + C::kCopiesPerTile) issue_one(m - 2);
                if (m == 2 + C::kCopiesPerTile) advance();
            }
#endif
            GPTOSS_FENCE();
        }
    };
    using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
    using T = std::true_type; using F = std::false_type;

    auto stage_tile = [&](int stage) { return smem_base + stage * (2 * kStageTileBytes); };
    auto stage_stat = [&](int stage) { return stat_base + stage * (2 * kTile * 4) + half * 16; };
    auto next_stage = [&](int stage) { return stage == NS - 1 ? 0 : stage + 1; };

    if (n_it > 0) {
        issue();
        issue();
        // The compiler does not see the copies (lds_dma16), but it does see this wait: from here on it knows
        // that the K / V loads above have arrived and puts no vmcnt wait of its own into the loop, where such
        // a wait would also drain the copies in flight.
        wait_vmcnt<0>();
        arrive();
        issue();
    }
    // one tile through the four slots (A..D of the header comment)
#ifdef GPTOSS_DKDV_TIMING
    uint64_t tsl[8] = {0, 0, 0, 0, 0, 0, 0, 0}, tprev = 0;
#define GPTOSS_TS(kk) { const uint64_t tnow = __builtin_readcyclecounter(); if (tprev) tsl[kk] += tnow - tprev; tprev = tnow; }
#else
#define GPTOSS_TS(kk)
#endif
    auto body = [&](auto masked_, uint32_t st, uint32_t stl, uint32_t nst, uint32_t nstl) __attribute__((always_inline)) {
        GPTOSS_TS(4)
        GPTOSS_FENCE();
        // slot A: M2(3 of the tile before), M1(1) | V(0) | block 1: statistics, natural fragments
        slot(masked_, I1{}, I3{}, I0{}, I1{}, I1{}, F{}, st, stl);
        GPTOSS_TS(0)
        // slot B: M2(0), M1(2) | V(1) | block 1: transposed fragments
        slot(masked_, I2{}, I0{}, I1{}, I2{}, I1{}, F{}, st, stl);
        GPTOSS_TS(1)
        // slot C: the next tile has landed (and this one's stage is free for the request after next);
        //         M2(1), M1(3) | V(2) | next tile, block 0: statistics, natural fragments
        // slot D: M2(2), M1(0 of the next tile) | V(3) | next tile, block 0: transposed fragments
        // (When the run ends here the next tile's part is still issued, on whatever the next stage holds:
        // staged data of a tile this wavefront skips, or a repeated copy after the last tile.  Its results
        // are never used; the body stays free of variants and branches.)
        slot(masked_, I3{}, I1{}, I2{}, I1{}, I0{}, T{}, nst, nstl);
        GPTOSS_TS(2)
        slot(masked_, I0{}, I2{}, I3{}, I2{}, I0{}, F{}, nst, nstl);
        GPTOSS_TS(3)
#ifdef GPTOSS_DKDV_TIMING
        tsl[5] += 1;
#endif
    };

    // A full-causal walk without padded rows (what the host sends here) meets, per wavefront: interior tiles,
    // then the masked tile(s) on the diagonal, then tiles whose rows all precede the wavefront's keys.  The
    // kernel is laid out as exactly that, one piece after the other with no loop around them.
    int k = 0;
    int cls = n_it > 0 ? classify(cur_i0) : kSkip;
    if (cls != kSkip) {
        // ---- the tiles that do something, through the pipeline ----
        {   // fill: block 0 of the first tile, M1(0).  The first slot of the loop also issues M2 of "the tile
            // before": for the first tile of a run that is a product of zeros (exact: the accumulators keep
            // their bits), which keeps the loop body free of variants.
            const uint32_t st = stage_tile(cur_stage), stl = stage_stat(cur_stage);
#pragma unroll
            for (int i = 0; i < 16; ++i) { s[3][i] = 0.0f; dp[3][i] = 0.0f; }
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
            for (int unit = 0; unit < 16; ++unit) rd(st, stl, 0, unit);
            GPTOSS_FENCE();
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                m1(0, j);
                rd(st, stl, 0, 16 + j);
                GPTOSS_FENCE();
            }
        }
        // The tiles of a run, interior ones first (as a causal layer's walk meets them), then masked ones; two
        // plain loops one after the other rather than one loop with two bodies, which the register allocator
        // cannot hold together.  The pipeline state passes from the first to the second.
        bool live = true;
        auto step_tile = [&](auto masked_) __attribute__((always_inline)) {
            const bool has_next = k + 1 < n_it;
            int n_h = cur_h + 1, n_i0 = cur_i0, ncls = cls;
            if (n_h == a.r) { n_h = 0; n_i0 -= kTile; ncls = has_next ? classify(n_i0) : kSkip; }
            const int nstage = next_stage(cur_stage);
            body(masked_, stage_tile(cur_stage), stage_stat(cur_stage), stage_tile(nstage), stage_stat(nstage));
            ++k;
            cur_stage = nstage;
            cur_h = n_h;
            cur_i0 = n_i0;
            cls = ncls;
            live = has_next && ncls != kSkip;
        };
        // (The explicit waits in front of the loops: whatever loads the compiler itself has in flight here,
        // reloads of spilled registers included, are then known to have arrived, and it puts no vmcnt wait of
        // its own into the loops, where it would drain the copies in flight on every pass.)
        wait_vmcnt<0>();
        while (live && cls == kInterior) step_tile(F{});
        if (live && cls == kMasked) {
            const int pos0 = q_offset + cur_i0;          // masked tiles that follow one another belong to one query tile
            const int row_lim = (int)min((int64_t)kTile, min((int64_t)a.Sq, (int64_t)q_len - q_offset) - cur_i0);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const int j = wj0 + 32 * nb + l32;
                const int dbase = (j < kv_len) ? pos0 - j : -0x40000000;
                mdb[nb] = dbase + 4 * half;
                mwd[nb] = (unsigned)max(0, min(weff, mdb[nb] + max(row_lim, -8) - 4 * half));
            }
            const int i0_masked = cur_i0;
            wait_vmcnt<0>();
            while (live && cls == kMasked && cur_i0 == i0_masked) step_tile(T{});
        }
        // drain: the tail of V(3) and M2(3)
        GPTOSS_FENCE();
        vstep(F{}, 3, 16);
        vstep(F{}, 3, 17);
        GPTOSS_FENCE();
#pragma unroll
        for (int j = 0; j < 8; ++j) m2(3, j);
        agpr_accumulators_settled(dk, dv);
    }
    // ---- the rest of the walk: nothing to compute, but every wavefront keeps the workgroup's rhythm of
    // barriers and requests ----
    for (; k < n_it; ++k) {
        arrive();
        issue();
    }
#undef GPTOSS_FENCE

#ifdef GPTOSS_DKDV_TIMING
    if (lane == 0 && blockIdx.x < 64) {
        float *dbg = a.delta + 2 * (int64_t)a.B * a.H * a.Sq + (blockIdx.x * 4 + w) * 8;
        for (int i = 0; i < 8; ++i) dbg[i] = (float)tsl[i];
    }
#endif
    wait_vmcnt<0>();          // the repeated copies of the last requests
    agpr_accumulators_settled(dk, dv);
    if (a.dkdv_parts > 1) {
        // unscaled fp32 partial sums; lane = key row, register i of block dblk = column 32*dblk + crow(i, half)
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
    bf16 *stage_out = reinterpret_cast<bf16 *>(&smem[0][0][0]) + w * 32 * kLS;
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
