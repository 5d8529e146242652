// Forward kernel: O = softmax([S, sink]) V without the sink column, plus the
// row logsumexp.  Stands in for the reference's `_attn_fwd`
// (attention_kernel.py:11-100).
//
// Work split.  A workgroup is 4 wavefronts.  Each wavefront owns 32*NQB query
// rows of ONE query head; the 4 wavefronts of a workgroup are HPB query heads of
// the same KV head times 4/HPB consecutive row slabs, so every K/V tile staged in
// LDS is shared by the whole GQA group slice.  KV tiles are 64 keys.
//
// Per tile the wavefront computes S^T = K Q^T (K rows are the MFMA A operand
// from LDS, Q^T lives in registers as the B operand), so a lane owns one query
// row per 32-row block and its logits sit in its own registers: the row max /
// row sum are in-lane reductions plus one exchange with lane^32.  exp2 is used
// with scale*log2(e) folded into one FMA.  P^T goes straight from the C
// registers into the B operand of O^T += V^T P^T; V^T fragments come from the
// row-major LDS tile through ds_read_b64_tr_b16.  With NQB = 2 every fragment
// read from LDS feeds two MFMAs.
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace gptoss {

// One 64-key tile for one wavefront.  MASKED = false: every pair visible.
// Masked variant: dbase[qb] = (lane's query position) - (first key of the tile),
// hugely negative for a dead query row; key r of the tile is visible iff
// 0 <= dbase - r < weff and r < key_lim.
template <bool MASKED, int NQB>
__device__ __forceinline__ void fwd_tile(uint32_t ksm, uint32_t vsm, const TileLaneOffsets &lo, const bf16x8 (&qf)[NQB][4],
                                         f32x16 (&o)[NQB][2], float (&m)[NQB], float (&l)[NQB], float c, int lane,
                                         const int (&dbase)[NQB], const unsigned (&wl)[NQB], unsigned weff, int key_lim,
                                         int wrel) {
    // wl[qb]: this lane's own window, min(window, distance back to the start of its document).
    // wrel (masked variant only): (first query position of the wavefront) - (first key of the
    // tile).  A 32-key half of the tile whose keys all lie in the future of every row of the
    // wavefront, or all fell out of every row's window, is skipped outright (no MFMA, no exp).
    const int half = lane >> 5;
    bool dead[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
        dead[kb] = MASKED && ((32 * kb > wrel + 32 * NQB - 1) || (32 * kb + 31 < wrel - (int)weff + 1) || (32 * kb >= key_lim));
    f32x16 s[2][NQB];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kb][qb][i] = dead[kb] ? -INFINITY : 0.0f;
        if (dead[kb]) continue;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 ak = ofrag_nat(ksm, lo, kb, ks);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb)
                s[kb][qb] = mfma_bf16(ak, qf[qb][ks], s[kb][qb]);
        }
    }
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        if (MASKED) {
            const KeyMask km = make_key_mask(dbase[qb], wl[qb], key_lim, half);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
                if (!dead[kb]) {
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        s[kb][qb][i] = key_visible(km, 32 * kb + 8 * (i >> 2) + (i & 3)) ? s[kb][qb][i] : -INFINITY;
                }
        }
        // two independent reduction chains keep the VALU pipelined
        float mx0 = s[0][qb][0], mx1 = s[1][qb][0];
#pragma unroll
        for (int i = 1; i < 16; ++i) { mx0 = fast_max(mx0, s[0][qb][i]); mx1 = fast_max(mx1, s[1][qb][i]); }
        float mx = fast_max(mx0, mx1);
        mx = xhalf_max(mx);
        const float m_new = fast_max(m[qb], mx * c);
        if (__builtin_amdgcn_ballot_w64(m_new != m[qb]) != 0ull) {
            const float alpha = fast_exp2(m[qb] - m_new);
            l[qb] *= alpha;
#pragma unroll
            for (int i = 0; i < 16; ++i) { o[qb][0][i] *= alpha; o[qb][1][i] *= alpha; }
            m[qb] = m_new;
        }
        float rs = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
            if (!dead[kb]) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float pe = fast_exp2(fmaf(s[kb][qb][i], c, -m[qb]));
                    s[kb][qb][i] = pe;
                    rs += pe;
                }
            }
        l[qb] += rs;
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        if (dead[kb]) continue;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bf16x8 av[2];
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) av[dblk] = ofrag_tr(vsm, lo, kb, u, dblk);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                const bf16x8 pf = cfrag(s[kb][qb], u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) o[qb][dblk] = mfma_bf16(av[dblk], pf, o[qb][dblk]);
            }
        }
    }
}

// The same tile with the softmax reference FROZEN: p = exp2(s*c + nm) with nm = -m, the lane's
// reference as the first tile of the row left it (the row maximum over that tile, or the sink
// logit if that is larger).  This is the reference's online softmax (attention_kernel.py:79-96)
// with the running maximum no longer updated: O = sum(p v) / (sum p + exp(sink - m)) is the same
// quotient for any m as long as nothing overflows, so after the first tile the key loop needs no
// row maximum, no comparison and no rescaling of O (in a sliding-window layer nearly every one
// of a row's three tiles moves the maximum and pays for that rescaling).  A row whose later
// logits climb more than about 95 (natural units) above its reference would overflow; the
// kernel detects that after the loop and repeats the workgroup with the exact step (fwd_tile)
// on every tile.  Logits far below the reference underflow to p = 0, which is what they
// contribute.  The row sum stays an fp32 sum of the unrounded probabilities, so lse is as
// exact as in fwd_tile.
template <bool MASKED, int NQB>
__device__ __forceinline__ void fwd_tile_lean(uint32_t ksm, uint32_t vsm, const TileLaneOffsets &lo, const bf16x8 (&qf)[NQB][4],
                                              f32x16 (&o)[NQB][2], const float (&nm)[NQB], float (&l)[NQB], float c, int lane,
                                              const int (&dbase)[NQB], const unsigned (&wl)[NQB], unsigned weff, int key_lim,
                                              int wrel) {
    const int half = lane >> 5;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        if (MASKED && ((32 * kb > wrel + 32 * NQB - 1) || (32 * kb + 31 < wrel - (int)weff + 1) || (32 * kb >= key_lim))) continue;
        f32x16 s[NQB];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[qb][i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 ak = ofrag_nat(ksm, lo, kb, ks);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) s[qb] = mfma_bf16(ak, qf[qb][ks], s[qb]);
        }
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            KeyMask km{0, 0u};
            if (MASKED) km = make_key_mask(dbase[qb], wl[qb], key_lim, half);
            float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                float t0 = fmaf(s[qb][i], c, nm[qb]), t1 = fmaf(s[qb][i + 1], c, nm[qb]);
                if (MASKED) {
                    t0 = key_visible(km, 32 * kb + 8 * (i >> 2) + (i & 3)) ? t0 : -INFINITY;
                    t1 = key_visible(km, 32 * kb + 8 * (i >> 2) + (i & 3) + 1) ? t1 : -INFINITY;
                }
                const float e0 = fast_exp2(t0), e1 = fast_exp2(t1);
                s[qb][i] = e0;
                s[qb][i + 1] = e1;
                rs0 += e0;
                rs1 += e1;
            }
            l[qb] += rs0 + rs1;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bf16x8 av[2];
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) av[dblk] = ofrag_tr(vsm, lo, kb, u, dblk);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                const bf16x8 pf = cfrag(s[qb], u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) o[qb][dblk] = mfma_bf16(av[dblk], pf, o[qb][dblk]);
            }
        }
    }
}

template <int HPB, int NQB>
__global__ __launch_bounds__(256, (NQB == 1 ? 3 : 2)) void attn_fwd_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    constexpr int QSUB = 4 / HPB;      // row slabs per workgroup
    constexpr int WM = 32 * NQB;       // query rows per wavefront
    constexpr int BM = WM * QSUB;      // query rows per workgroup
    constexpr int NS = 3;              // LDS stages: K/V tiles are requested two iterations ahead
    __shared__ __attribute__((aligned(16))) char smem[NS][2][kStageTileBytes];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;

    // workgroup -> (kv head, head chunk, batch, query tile); the kv head is the
    // fastest index so that with G == 8 each XCD (workgroups are dealt round-robin
    // over the 8 XCDs) keeps one KV head's K/V in its own L2.  Query tiles run from
    // the last (longest key loop) to the first.
    const int n_hc = (a.r + HPB - 1) / HPB;
    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int hc = bid % n_hc; bid /= n_hc;
    const int b = bid % a.B; bid /= a.B;
    const int n_qt = (a.Sq + BM - 1) / BM;
    const int qt = n_qt - 1 - bid;

    const int hsel = hc * HPB + (w % HPB);
    const bool active = hsel < a.r;
    const int head = g * a.r + (active ? hsel : 0);
    const int qw0 = qt * BM + WM * (w / HPB);          // first query row of this wavefront

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window ? a.window : 0x3fffffff;

    // key range of the workgroup (union over its wavefronts)
    const int bpos0 = q_offset + qt * BM;
    const int bpos1 = min(q_offset + min(a.Sq, (qt + 1) * BM) - 1, q_len - 1);
    const int hi = bpos1 >= bpos0 ? min(kv_len, bpos1 + 1) : 0;   // no key at all for a fully padded tile
    const int key_lo = max(0, bpos0 - weff + 1);
    // packed rows: first key of the document of the workgroup's first row (document starts never
    // decrease along a row), and of this wavefront's first and last rows
    const int32_t *dsrow = a.doc_start ? a.doc_start + (int64_t)b * a.Sq : nullptr;
    const int ds_b0 = dsrow ? dsrow[min(qt * BM, a.Sq - 1)] : 0;
    const int ds_w0 = dsrow ? dsrow[min(qw0, a.Sq - 1)] : 0;
    const int ds_w1 = dsrow ? dsrow[min(qw0 + WM - 1, a.Sq - 1)] : 0;
    const int t_lo = max(key_lo, ds_b0) / kTile;
    const int t_hi = hi > 0 ? (hi + kTile - 1) / kTile : 0;

    // this wavefront's own row range (absolute positions)
    // (wave-uniform values, said so to the compiler: the tile classification below then branches
    // on scalar conditions)
    const int wpos0 = __builtin_amdgcn_readfirstlane(q_offset + qw0);
    const int wpos1 = __builtin_amdgcn_readfirstlane(min(q_offset + min(a.Sq, qw0 + WM) - 1, q_len - 1));

    const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const bf16 *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;

    // Q^T fragments (B operand), resident for the whole key loop
    bf16x8 qf[NQB][4];
    int pq[NQB];            // lane's query position per block, hugely negative when the row is dead
    unsigned wl[NQB];       // lane's own window: min(window, distance back to its document's first key)
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int row = qw0 + 32 * qb + l32;
        const bf16 *qrow = a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)row * a.qs.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 z = {0u, 0u, 0u, 0u};
            if (row < a.Sq) z = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * half);
            qf[qb][ks] = as_bf16x8(z);
        }
        const int p = q_offset + row;
        pq[qb] = (row < a.Sq && p < q_len) ? p : -0x40000000;
        wl[qb] = (unsigned)weff;
        if (dsrow && row < a.Sq) wl[qb] = (unsigned)min(weff, p - dsrow[row] + 1);
    }

    const float c = a.scale_log2;
    const float sink2 = (a.sinks ? a.sinks[head] : 0.0f) * kLog2e;
    float m[NQB], l[NQB];  // softmax reference (log2 domain, starts at the sink logit, ref :53) and
                           // this lane's share of the running sum (own keys only)
    f32x16 o[NQB][2];

    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(&smem[0][0][0]);
    const int n_it = max(0, t_hi - t_lo);
    // K / V tiles are requested in order; the pointers to the next tile's first row advance by
    // one tile per request.  Only a tile that sticks out of the tensor takes the clamping copy.
    const AsyncLaneOffsets klane = make_async_offsets(a.ks.s, lane, w), vlane = make_async_offsets(a.vs.s, lane, w);
    const int w_s = __builtin_amdgcn_readfirstlane(w);
    const bf16 *ktile = kbase, *vtile = vbase;
    int next_row0 = 0;
    auto issue = [&](int it) __attribute__((always_inline)) {
        const int stage = it % NS;
        if (next_row0 + kTile <= a.Skv) {
            tile_async_inner(smem[stage][0], ktile, klane, w_s);      // (scalar wave index: the LDS base is formed on the scalar unit)
            tile_async_inner(smem[stage][1], vtile, vlane, w_s);
        } else {
            tile_async(smem[stage][0], kbase, a.ks.s, next_row0, a.Skv, lane, w);
            tile_async(smem[stage][1], vbase, a.vs.s, next_row0, a.Skv, lane, w);
        }
        ktile += kTile * a.ks.s;
        vtile += kTile * a.vs.s;
        next_row0 += kTile;
    };
    constexpr int kLoadsPerIt = 4;     // vector-memory instructions one wavefront issues per iteration

    // (re)starts the walk over the workgroup's key tiles
    auto reset = [&]() __attribute__((always_inline)) {
        ktile = kbase + (int64_t)t_lo * kTile * a.ks.s;
        vtile = vbase + (int64_t)t_lo * kTile * a.vs.s;
        next_row0 = t_lo * kTile;
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            m[qb] = sink2;
            l[qb] = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) { o[qb][0][i] = 0.0f; o[qb][1][i] = 0.0f; }
        }
        if (n_it > 0) issue(0);
        if (n_it > 1) issue(1);
    };
    // the synchronisation every iteration starts with: this tile's copies have landed in every
    // wavefront, the stage two tiles ahead is free
    auto arrive = [&](int it) __attribute__((always_inline)) {
        if (it + 1 < n_it) wait_vmcnt<kLoadsPerIt>(); else wait_vmcnt<0>();
        __syncthreads();
        if (it + 2 < n_it) issue(it + 2);
    };
    // One key tile from the LDS stage at ksm.  EXACT: the online-softmax step that moves the
    // reference m (fwd_tile); otherwise m stays where it is (fwd_tile_lean).
    auto tile_step = [&](int it, uint32_t ksm, auto exact_tag) __attribute__((always_inline)) {
        constexpr bool EXACT = decltype(exact_tag)::value;
        const uint32_t vsm = ksm + kStageTileBytes;
        const int n0 = (t_lo + it) * kTile;
        // tile classification for this wavefront: skip / interior / needs mask
        const bool skip = !active || n0 > wpos1 || (n0 + kTile - 1) < (wpos0 - weff + 1) || wpos1 < wpos0 ||
                          (n0 + kTile - 1) < ds_w0;
        if (skip) return;
        const bool interior = (n0 + kTile - 1 <= wpos0) && (n0 > wpos1 - weff) && (n0 + kTile <= kv_len) &&
                              (q_offset + qw0 + WM - 1 <= wpos1) && (n0 >= ds_w1);
        int dbase[NQB];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) dbase[qb] = pq[qb] - n0;   // stays hugely negative for dead rows
        if constexpr (EXACT) {
            if (interior) fwd_tile<false, NQB>(ksm, vsm, lo, qf, o, m, l, c, lane, pq, wl, 0u, 0, 0);
            else fwd_tile<true, NQB>(ksm, vsm, lo, qf, o, m, l, c, lane, dbase, wl, (unsigned)weff, kv_len - n0, wpos0 - n0);
        } else {
            float nm[NQB];
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) nm[qb] = -m[qb];
            if (interior) fwd_tile_lean<false, NQB>(ksm, vsm, lo, qf, o, nm, l, c, lane, pq, wl, 0u, 0, 0);
            else fwd_tile_lean<true, NQB>(ksm, vsm, lo, qf, o, nm, l, c, lane, dbase, wl, (unsigned)weff, kv_len - n0, wpos0 - n0);
        }
    };
    // Long full-causal rows (64-row wavefronts) freeze the reference after their first tile.  The
    // 32-row wavefronts of sliding-window layers keep the exact step on all of their three tiles:
    // measured, the frozen form does not pay there (0.099 -> 0.103 ms at S = 16384), and with so
    // few keys per row a dominant key met after the first tile (weights above 1 in the numerator,
    // bf16-rounded there but not in the denominator) shows in dQ of sharply peaked rows.
    constexpr bool kFreeze = NQB == 2;
    auto lean_step = [&](int it, auto stage_tag) __attribute__((always_inline)) {
        constexpr int STAGE = decltype(stage_tag)::value;
        arrive(it);
        tile_step(it, smem_base + STAGE * (2 * kStageTileBytes), std::integral_constant<bool, !kFreeze>{});
    };

    // Main pass, unrolled by LDS stage so that every fragment address is (per-lane offset
    // register) + (immediate).  With kFreeze the first tile runs the exact step and sets every
    // lane's reference, the others keep it frozen.
    reset();
    if constexpr (kFreeze) {
        if (n_it > 0) {
            arrive(0);
            tile_step(0, smem_base, std::true_type{});
        }
        for (int it = 1; it < n_it; it += NS) {
            lean_step(it, std::integral_constant<int, 1>{});
            if (it + 1 < n_it) lean_step(it + 1, std::integral_constant<int, 2>{});
            if (it + 2 < n_it) lean_step(it + 2, std::integral_constant<int, 0>{});
        }
    } else {
        for (int it = 0; it < n_it; it += NS) {
            lean_step(it, std::integral_constant<int, 0>{});
            if (it + 1 < n_it) lean_step(it + 1, std::integral_constant<int, 1>{});
            if (it + 2 < n_it) lean_step(it + 2, std::integral_constant<int, 2>{});
        }
    }
    // A sum beyond 2^96 (or not finite) means some logit stood some 95 or more above its row's
    // reference and the products may have overflowed: the workgroup repeats its key loop with the
    // exact step on every tile (rare, so this pass has one loop body with a run-time LDS stage).
    bool unsafe = false;
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) unsafe = unsafe || !(l[qb] < 0x1p96f);
    if (kFreeze && __syncthreads_or(unsafe)) {
        reset();
        int stage = 0;
        for (int it = 0; it < n_it; ++it) {
            arrive(it);
            tile_step(it, smem_base + stage * (2 * kStageTileBytes), std::true_type{});
            stage = stage == NS - 1 ? 0 : stage + 1;
        }
    }

    // epilogue: z = l + exp(sink - m); O = acc / z; M = m + log z   (ref :93-98)
    __syncthreads();   // every wavefront is done reading the K/V buffers
    bf16 *stage = reinterpret_cast<bf16 *>(&smem[0][0][0]) + w * 32 * kLS;
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const float l_tot = l[qb] + __shfl_xor(l[qb], 32);
        const float z = l_tot + fast_exp2(sink2 - m[qb]);
        const float inv = 1.0f / z;
        if (active) {
            const int r0 = qw0 + 32 * qb;
            bf16 *orow0 = a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)r0 * a.os.s;
            store_rows32(stage, o[qb], inv, orow0, a.os.s, a.Sq - r0, lane);
            __builtin_amdgcn_wave_barrier();
            if (half == 0 && r0 + l32 < a.Sq)
                a.lse[((int64_t)b * a.H + head) * a.Sq + r0 + l32] = (m[qb] + fast_log2(z)) * kLn2;
        }
    }
}

}  // namespace gptoss
