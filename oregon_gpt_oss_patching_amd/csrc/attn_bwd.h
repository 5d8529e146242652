// Backward kernels.  Together they stand in for the reference's
// `_attn_bwd_precompute_D` (attention_kernel.py:102-120) and `_attn_bwd`
// (:122-217), split so that no gradient needs an atomic:
//   attn_bwd_delta_kernel   delta = rowsum(dO * O)                      (:119)
//   attn_bwd_dsinks_kernel  dsinks[h] = -sum exp(sink - M) * delta      (:173-176)
//   attn_bwd_dkdv_kernel    KV-outer: a workgroup owns 128 keys of one KV head
//                           and walks every (query head of the group, query
//                           tile) that can see them                      (:199-212)
//   attn_bwd_dq_kernel      Q-outer, same shape as the forward kernel    (:206-217)
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace gptoss {

// ---------------------------------------------------------------------------------
// -delta[b,h,s] = -sum_d dO[b,h,s,d] * O[b,h,s,d] (negated so that the dK/dV kernel can
// load it straight into the dP accumulators).  HBM-bound stream: eight lanes
// read one 128-byte row of each tensor, reduce with three xor-shuffles.  The same
// pass stores lse*log2(e) in the second half of the scratch buffer, which is what
// the dQ and dSinks kernels feed to exp2, and both statistics once more in the split form the
// dK/dV kernels take (split_row_stats).
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(const KArgs a) {
    constexpr int kRowsPerThread = 4;                      // independent 128-bit loads in flight per tensor
    const int64_t total = (int64_t)a.B * a.H * a.Sq;       // rows, indexed (b*H + h)*Sq + s
    const int c = threadIdx.x & 7;
    const int64_t rid0 = (int64_t)blockIdx.x * (32 * kRowsPerThread) + (threadIdx.x >> 3);
    u32x4 ov[kRowsPerThread], gv[kRowsPerThread];
#pragma unroll
    for (int k = 0; k < kRowsPerThread; ++k) {
        const int64_t rid = rid0 + 32 * k;
        ov[k] = u32x4{0u, 0u, 0u, 0u};
        gv[k] = u32x4{0u, 0u, 0u, 0u};
        if (rid < total) {
            const int s = (int)(rid % a.Sq);
            const int bh = (int)(rid / a.Sq);
            const int h = bh % a.H, b = bh / a.H;
            ov[k] = *reinterpret_cast<const u32x4 *>(a.o + (int64_t)b * a.os.b + (int64_t)h * a.os.h + (int64_t)s * a.os.s + c * 8);
            gv[k] = *reinterpret_cast<const u32x4 *>(a.d_o + (int64_t)b * a.dos.b + (int64_t)h * a.dos.h + (int64_t)s * a.dos.s + c * 8);
        }
    }
#pragma unroll
    for (int k = 0; k < kRowsPerThread; ++k) {
        const int64_t rid = rid0 + 32 * k;
        const bf16x8 of = as_bf16x8(ov[k]), gf = as_bf16x8(gv[k]);
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc = fmaf((float)of[j], (float)gf[j], acc);
        acc += __shfl_xor(acc, 1);
        acc += __shfl_xor(acc, 2);
        acc += __shfl_xor(acc, 4);
        if (c == 0 && rid < total) {
            a.delta[rid] = -acc;                          // stored negated: it seeds the dP accumulators
            a.delta[total + rid] = a.lse[rid] * kLog2e;   // second half of the scratch: lse in log2 units
            a.split[rid] = split_row_stats(a.lse[rid], a.scale, -acc);
        }
    }
}

// ---------------------------------------------------------------------------------
// One workgroup per query head; fixed summation order, so the result is
// bit-reproducible (the reference accumulates it with relaxed atomics).
__global__ __launch_bounds__(1024) void attn_bwd_dsinks_kernel(const KArgs a) {
    __shared__ float red[1024];
    const int h = blockIdx.x;
    const float sink2 = (a.sinks ? a.sinks[h] : 0.0f) * kLog2e;
    const int64_t total = (int64_t)a.B * a.H * a.Sq;
    float acc = 0.0f;
    for (int b = 0; b < a.B; ++b) {
        const float *ndl = a.delta + ((int64_t)b * a.H + h) * a.Sq;        // -delta
        const float *lse2 = ndl + total;                                    // lse * log2(e)
        for (int s = threadIdx.x; s < a.Sq; s += 1024) acc += fast_exp2(sink2 - lse2[s]) * ndl[s];
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int off = 512; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) a.dsinks[h] = red[0];
}

// ---------------------------------------------------------------------------------
// dS exchange through LDS (fused backward).  The dS tile is key-major: key row r of the
// workgroup occupies 128 bytes (64 query-row columns in bf16), chunk-swizzled by swz(r).
// A lane of an owner wavefront (key row r, half = lane / 32) holds, per 16-row step u of the
// 32-row block qb, the B fragment dsf: elements 0..3 are rows 16u + 4*half + 0..3, elements 4..7
// rows 16u + 8 + 4*half + 0..3, i.e. two 8-byte pieces in the logical chunks 4*qb + 2*u and
// 4*qb + 2*u + 1 of its key row, at byte 8*half of the chunk.  With the row's swizzle folded into
// the base address the chunk selection is one XOR with an immediate.
__device__ __forceinline__ uint32_t ds_store_addr(uint32_t tile, int keyrow, int half) {
    return tile + keyrow * kRowBytes + (swz(keyrow) << 4) + 8 * half;
}
__device__ __forceinline__ void ds_store(uint32_t base, int qb, int u, const bf16x8 dsf) {
    typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
    bf16x4 p0, p1;
#pragma unroll
    for (int e = 0; e < 4; ++e) { p0[e] = dsf[e]; p1[e] = dsf[4 + e]; }
    *reinterpret_cast<lds_bf16x4 *>((uintptr_t)(base ^ ((4 * qb + 2 * u) << 4))) = p0;
    *reinterpret_cast<lds_bf16x4 *>((uintptr_t)(base ^ ((4 * qb + 2 * u + 1) << 4))) = p1;
}
__device__ __forceinline__ void ds_store_zero(uint32_t base, int qb) {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (bf16)0.0f;
    ds_store(base, qb, 0, z);
    ds_store(base, qb, 1, z);
}

// ---- MFMAs whose accumulator lives in the AGPR half of the register file -----------------------------
// A kernel that runs one wavefront per SIMD has 512 registers per lane, 256 of them AGPRs, which only
// MFMAs (and copies) can touch.  The compiler keeps all MFMA results of a kernel in one kind of register;
// the library is built so that this is the VGPR kind (the vector instructions of the softmax read S and
// dP), and the long-lived dK / dV accumulators of attn_bwd_dkdv64_kernel are kept in AGPRs through these
// inline-assembly MFMAs.  What the compiler cannot see inside the assembly, and the callers therefore
// guarantee themselves:
//   * an operand written by a vector instruction is at least two instructions old when the MFMA reads it
//     (SAFE pays for that itself with two wait states);
//   * no other instruction reads an accumulator sooner than an MFMA takes to finish, not even a
//     register-to-register copy, which the compiler may place wherever two pieces of straight-line code
//     meet (it does move the accumulators between the pipelined loop and the code around it): the last
//     of these MFMAs in such a piece is followed by eight or more ordinary MFMAs or by
//     agpr_accumulators_settled(), and the first one in a piece is the SAFE form (a copy is a vector
//     instruction too).  tests/test_isa_dkdv64.py checks the compiled kernel for this.
template <bool SAFE>
__device__ __forceinline__ void mfma_bf16_agpr(f32x16 &acc, const bf16x8 a, const bf16x8 b) {
    if constexpr (SAFE) asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    else asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// Longer than the 16 passes of the slowest MFMA.  The accumulators are operands, so they are still where
// the MFMAs left them when the delay starts and anything the compiler does with them comes after it.
__device__ __forceinline__ void agpr_accumulators_settled(f32x16 (&dk)[2][2], f32x16 (&dv)[2][2]) {
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15"
                 : "+a"(dv[0][0]), "+a"(dv[0][1]), "+a"(dv[1][0]), "+a"(dv[1][1]), "+a"(dk[0][0]), "+a"(dk[0][1]), "+a"(dk[1][0]),
                   "+a"(dk[1][1]));
}

// ---------------------------------------------------------------------------------
// dK, dV.  Workgroup = NW wavefronts x 64 keys of KV head g, batch b.  The K and V
// rows of a wavefront stay in registers as MFMA B operands (two 32-key blocks, so
// every Q / dO fragment fetched from LDS feeds two MFMAs).  The loop streams
// 64-row Q and dO tiles (plus their lse / delta) of each of the r query heads
// through LDS:
//   S  = Q K^T, dP = dO V^T         (A = Q / dO rows from LDS, natural reads)
//   P  = exp2(S*c - lse*log2e),  dS = P * (dP - delta)
//   dV^T += dO^T P,  dK^T += Q^T dS (A = transposed LDS reads, B = C registers)
// A lane owns two keys; accumulators are written once at the end.
// One 64-row query tile against a wavefront's 64 keys (see attn_bwd_dkdv_kernel).
// MASKED = false is the interior fast path: every (query, key) pair is visible.
// In the masked variant `dbase[nb]` is (first query position of the tile) - (this
// lane's key), or a huge negative number for a dead key, so that pair (row r, key)
// is visible iff 0 <= dbase + r < weff, tested with one unsigned compare; rows at
// or beyond `row_lim` (relative to the tile) do not exist.
// STORE_DS (needs NB == 1): the bf16 dS values of the tile are also written to LDS, key-major: the
// lane's key row starts at ds_out (which already holds the row's swizzle, see ds_store_addr), one
// 128-byte row of 64 query-row columns per key, 16-byte chunks XOR-swizzled like every staged
// tile.  A 32-row block that is skipped stores zeros.  The wavefronts that form dQ read it back
// with the transposing fragment reads.
// SPLIT: the row statistics are staged in the split form (split_row_stats) and enter through one more
// step of the S and dP contractions; stat_lane then addresses the 16 bytes of row l32 of block 0.
template <bool MASKED, bool DOCS, int NB, bool STORE_DS = false, bool SPLIT = false>
__device__ __forceinline__ void dkdv_tile(uint32_t qsm, uint32_t gsm, uint32_t stat_lane, const TileLaneOffsets &lo,
                                          const bf16x8 (&kf)[NB][4], const bf16x8 (&vf)[NB][4],
                                          f32x16 (&dk)[NB][2], f32x16 (&dv)[NB][2], float c, int half,
                                          const int (&dbase)[NB], unsigned weff, int row_lim, int krel,
                                          uint32_t ds_lane, const int (&jkey)[NB], uint32_t ds_out = 0) {
    static_assert(!STORE_DS || NB == 1, "the dS store is written for one 32-key block per wavefront");
    // masked variant, per lane and tile: pair (row r, key) is visible iff 0 <= dbase + r < weff and
    // r < row_lim.  With r = rc + 4*half (rc a compile-time constant per accumulator register) that is
    // (unsigned)(dbh + rc) < width with dbh = dbase + 4*half, width = max(0, min(weff, dbh + row_lim - 4*half)):
    // one add, one compare, one select per element.  Used by the single-pass window kernel, where
    // two tiles out of three are masked (window layer, S = 16384: -6 %); the dK/dV kernel, whose
    // masked tiles are the few on the diagonal of a full-causal layer, keeps the plain form (the
    // folded one costs it 17 registers and 4 % on that layer).
    int dbh[NB];
    unsigned width[NB];
    if (MASKED && STORE_DS) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            dbh[nb] = dbase[nb] + 4 * half;
            width[nb] = (unsigned)max(0, min((int)weff, dbh[nb] + max(row_lim, -8) - 4 * half));
        }
    }
    bf16x8 b_stat_s, b_stat_dp;
    if constexpr (SPLIT) stat_step_operands(half, b_stat_s, b_stat_dp);
    // qsm / gsm: LDS byte addresses of the staged Q and dO tiles; stat_lane (not SPLIT): address of this
    // lane's first lse2 value (rows 4*half..), -delta sits kTile floats further on.
    // DOCS (packed rows): ds_lane addresses the staged document starts of the same rows, jkey
    // is the lane's key index; a key before its query's document start is invisible.
    // krel (masked variant only): (first key of the wavefront) - (first query position of the
    // tile); a 32-row block whose rows all precede the keys, or all lost them from their
    // window, is skipped.
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        if (MASKED && ((32 * qb + 31 < krel) || (32 * qb > krel + 32 * NB - 1 + (int)weff - 1) || (32 * qb >= row_lim))) {
            if constexpr (STORE_DS) ds_store_zero(ds_out, qb);
            continue;
        }
        f32x16 s[NB], dp[NB];
        if constexpr (SPLIT) {
            // the statistics step: S starts at -lse / scale, dP at -delta of the rows
            const bf16x8 a_stat = as_bf16x8(lds_load128(stat_lane, 32 * qb * 16));
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
                for (int i = 0; i < 16; ++i) { s[nb][i] = 0.0f; dp[nb][i] = 0.0f; }
                s[nb] = mfma_bf16(a_stat, b_stat_s, s[nb]);
                dp[nb] = mfma_bf16(a_stat, b_stat_dp, dp[nb]);
            }
        } else {
            // the dP accumulators start at -delta of their rows, so the MFMAs deliver dP - delta
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const f32x4 nd = lds_load128f(stat_lane, (kTile + 32 * qb + 8 * a4) * 4);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) { s[nb][4 * a4 + e] = 0.0f; dp[nb][4 * a4 + e] = nd[e]; }
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 aq = ofrag_nat(qsm, lo, qb, ks);
            const bf16x8 ag = ofrag_nat(gsm, lo, qb, ks);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                s[nb] = mfma_bf16(aq, kf[nb][ks], s[nb]);
                dp[nb] = mfma_bf16(ag, vf[nb][ks], dp[nb]);
            }
        }
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            f32x4 lv = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (!SPLIT) lv = lds_load128f(stat_lane, (32 * qb + 8 * a4) * 4);
            u32x4 dsr = {0u, 0u, 0u, 0u};
            if (MASKED && DOCS) dsr = lds_load128(ds_lane, (32 * qb + 8 * a4) * 4);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 4 * a4 + e;
                    float pe = fast_exp2(SPLIT ? s[nb][i] * c : fmaf(s[nb][i], c, -lv[e]));
                    if (MASKED) {
                        bool vis;
                        if constexpr (STORE_DS) {
                            vis = (unsigned)(dbh[nb] + (32 * qb + 8 * a4 + e)) < width[nb];
                        } else {
                            const int r = 32 * qb + 8 * a4 + 4 * half + e;
                            vis = ((unsigned)(dbase[nb] + r) < weff) & (r < row_lim);
                        }
                        if (DOCS) vis = vis & (jkey[nb] >= (int)dsr[e]);
                        pe = vis ? pe : 0.0f;
                    }
                    s[nb][i] = pe;
                    dp[nb][i] = pe * dp[nb][i];
                }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bf16x8 agt[2], aqt[2];
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) {
                agt[dblk] = ofrag_tr(gsm, lo, qb, u, dblk);
                aqt[dblk] = ofrag_tr(qsm, lo, qb, u, dblk);
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const bf16x8 pf = cfrag(s[nb], u), dsf = cfrag(dp[nb], u);
                if constexpr (STORE_DS) ds_store(ds_out, qb, u, dsf);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) {
                    dv[nb][dblk] = mfma_bf16(agt[dblk], pf, dv[nb][dblk]);
                    dk[nb][dblk] = mfma_bf16(aqt[dblk], dsf, dk[nb][dblk]);
                }
            }
        }
    }
}

template <int NW, int NB, bool DOCS>  // NB = 32-key blocks per wavefront; DOCS = packed rows (doc_start given)
__global__ __launch_bounds__(NW * 64, (NB == 1 ? 2 : 1)) void attn_bwd_dkdv_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    static_assert(NW == 4, "the asynchronous tile copy is written for 4 wavefronts");
    constexpr int NS = 3;              // LDS stages: tiles are requested two iterations ahead
    constexpr int WK = 32 * NB;        // keys per wavefront
    constexpr int BN = WK * NW;        // keys per workgroup
    __shared__ __attribute__((aligned(16))) char smem[NS][2][kStageTileBytes];
    __shared__ __attribute__((aligned(16))) u32x4 sstat[NS][kTile];               // split row statistics of the staged rows
    __shared__ __attribute__((aligned(16))) int32_t sdoc[DOCS ? NS : 1][kTile];   // document starts of the staged rows

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
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

    // query rows that can see any key of the workgroup
    const int j1 = min(j0 + BN, kv_len) - 1;              // last live key
    const int i_lo = max(0, j0 - q_offset);
    int64_t i_hi64 = min((int64_t)a.Sq, (int64_t)q_len - q_offset);
    i_hi64 = min(i_hi64, (int64_t)j1 + weff - q_offset);
    const int i_hi = (j1 >= j0) ? (int)max((int64_t)0, i_hi64) : 0;
    // With dkdv_parts > 1 the query tiles of the key block (walked from the last one down) are cut
    // into dkdv_parts consecutive slices, one per workgroup; each leaves an fp32 partial sum and
    // attn_bwd_dkdv_reduce_kernel adds them in a fixed order.
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

    f32x16 dk[NB][2], dv[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) { dk[nb][0][i] = dk[nb][1][i] = 0.0f; dv[nb][0][i] = dv[nb][1][i] = 0.0f; }

    const float c = a.scale_log2;
    int dead[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) dead[nb] = 0;
    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(&smem[0][0][0]), stat_base = lds_addr(&sstat[0][0]);
    const uint32_t doc_base = lds_addr(&sdoc[0][0]);
    constexpr bool has_docs = DOCS;
    int jkey[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) jkey[nb] = wj0 + 32 * nb + l32;

    // Iteration `it` -> (query tile, query head).  Query tiles run from the LAST one
    // down and heads are the inner index, so every workgroup of this KV head that is
    // resident at the same time walks the same Q / dO tiles in the same order and finds
    // them in its XCD's L2.  The walk is kept as running pointers (one step per request):
    // no division or 64-bit multiplication in the loop.
    const AsyncLaneOffsets qlane = make_async_offsets(a.qs.s, lane, w), glane = make_async_offsets(a.dos.s, lane, w);
    int iss_h = 0, iss_i0 = (qt_hi - 1) * kTile;                      // head within the group, first row of the tile
    const bf16 *qtile = a.q + (int64_t)b * a.qs.b + (int64_t)(g * a.r) * a.qs.h + (int64_t)iss_i0 * a.qs.s;
    const bf16 *gtile = a.d_o + (int64_t)b * a.dos.b + (int64_t)(g * a.r) * a.dos.h + (int64_t)iss_i0 * a.dos.s;
    int64_t stat_off = ((int64_t)b * a.H + (int64_t)g * a.r) * a.Sq + iss_i0;    // (b, head, row) of the tile's first row
    // wavefront w copies the statistics of 16 rows (16 bytes each) per tile, and 16 document starts
    const u32x4 *stat_lane = a.split + 16 * w + (lane & 15);
    const int32_t *doc_lane = DOCS ? a.doc_start + (int64_t)b * a.Sq + 16 * w + (lane & 15) : nullptr;
    auto issue = [&](int it) {
        const int stage = it % NS;
        if (iss_i0 + kTile <= a.Sq) {
            tile_async_inner(smem[stage][0], qtile, qlane, w);
            tile_async_inner(smem[stage][1], gtile, glane, w);
            if (lane < 16)
                __builtin_amdgcn_global_load_lds((glb_void_t *)(stat_lane + stat_off), (lds_void_t *)(&sstat[stage][16 * w]), 16, 0, 0);
            if (DOCS && lane < 16)
                __builtin_amdgcn_global_load_lds((glb_void_t *)(doc_lane + iss_i0), (lds_void_t *)(&sdoc[DOCS ? stage : 0][16 * w]), 4, 0, 0);
        } else {
            // the tile sticks out of the tensor: rows past the end re-read the last valid one
            tile_async(smem[stage][0], qtile - (int64_t)iss_i0 * a.qs.s, a.qs.s, iss_i0, a.Sq, lane, w);
            tile_async(smem[stage][1], gtile - (int64_t)iss_i0 * a.dos.s, a.dos.s, iss_i0, a.Sq, lane, w);
            if (lane < 16) {
                const int over = max(0, iss_i0 + 16 * w + lane - (a.Sq - 1));
                __builtin_amdgcn_global_load_lds((glb_void_t *)(stat_lane + stat_off - over), (lds_void_t *)(&sstat[stage][16 * w]), 16, 0, 0);
            }
            if (DOCS && lane < 16) {
                const int over = max(0, iss_i0 + 16 * w + lane - (a.Sq - 1));
                __builtin_amdgcn_global_load_lds((glb_void_t *)(doc_lane + iss_i0 - over), (lds_void_t *)(&sdoc[DOCS ? stage : 0][16 * w]), 4, 0, 0);
            }
        }
        ++iss_h;
        qtile += a.qs.h;
        gtile += a.dos.h;
        stat_off += a.Sq;
        if (iss_h == a.r) {
            iss_h = 0;
            iss_i0 -= kTile;
            qtile -= (int64_t)a.r * a.qs.h + (int64_t)kTile * a.qs.s;
            gtile -= (int64_t)a.r * a.dos.h + (int64_t)kTile * a.dos.s;
            stat_off -= (int64_t)a.r * a.Sq + kTile;
        }
    };
    int cur_h = 0, cur_i0 = (qt_hi - 1) * kTile;                      // the same walk for the tile being consumed
    // vector-memory instructions one wavefront issues per iteration: 5, or 6 with document starts

    // One iteration on a compile-time LDS stage, so that every fragment address is
    // (lane offset register) + (immediate).
    auto iterate = [&](int it, auto stage_tag) {
        constexpr int STAGE = decltype(stage_tag)::value;
        // the copies for this iteration were issued two iterations ago; those of the next
        // one may stay in flight
        if (it + 1 >= n_it) wait_vmcnt<0>(); else if (has_docs) wait_vmcnt<6>(); else wait_vmcnt<5>();
        __syncthreads();
        if (it + 2 < n_it) issue(it + 2);

        const uint32_t qsm = smem_base + STAGE * (2 * kStageTileBytes), gsm = qsm + kStageTileBytes;
        const uint32_t stat_lane = stat_base + STAGE * (kTile * 16) + l32 * 16;
        const uint32_t ds_lane = doc_base + STAGE * (kTile * 4) + half * 16;
        const int i0 = cur_i0;
        if (++cur_h == a.r) { cur_h = 0; cur_i0 -= kTile; }
        const int pos0 = q_offset + i0;                                    // first query position of the tile
        const int pos1 = min(q_offset + min(a.Sq, i0 + kTile) - 1, q_len - 1);   // last live one
        const int wj1 = min(wj0 + WK, kv_len) - 1;                           // wavefront's last live key
        bool skip = wj1 < wj0 || pos1 < wj0 || pos0 > wj1 + weff - 1 || pos1 < pos0;
        bool interior = (wj0 + WK - 1 <= pos0) && (wj0 > pos1 - weff) && (wj0 + WK <= kv_len) &&
                        (q_offset + i0 + kTile - 1 <= pos1);
        if constexpr (DOCS) {
            // document starts never decrease along a row: the tile's first row has the smallest,
            // its last row the largest (rows past the end repeat the last valid one)
            const int ds_first = __builtin_amdgcn_readfirstlane(sdoc[STAGE][0]);
            const int ds_last = __builtin_amdgcn_readfirstlane(sdoc[STAGE][kTile - 1]);
            skip = skip || ds_first > wj1;
            interior = interior && ds_last <= wj0;
        }
        if (skip) return;
        if (interior) {
            dkdv_tile<false, false, NB, false, true>(qsm, gsm, stat_lane, lo, kf, vf, dk, dv, c, half, dead, 0u, 0, 0, 0u, jkey);
        } else {
            int dbase[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const int j = wj0 + 32 * nb + l32;
                dbase[nb] = (j < kv_len) ? pos0 - j : -0x40000000;
            }
            const int row_lim = (int)min((int64_t)kTile, min((int64_t)a.Sq, (int64_t)q_len - q_offset) - i0);
            dkdv_tile<true, DOCS, NB, false, true>(qsm, gsm, stat_lane, lo, kf, vf, dk, dv, c, half, dbase, (unsigned)weff, row_lim,
                                      wj0 - pos0, ds_lane, jkey);
        }
    };

    if (n_it > 0) issue(0);
    if (n_it > 1) issue(1);
    for (int it = 0; it < n_it; it += NS) {
        iterate(it, std::integral_constant<int, 0>{});
        if (it + 1 < n_it) iterate(it + 1, std::integral_constant<int, 1>{});
        if (it + 2 < n_it) iterate(it + 2, std::integral_constant<int, 2>{});
    }

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

// ---------------------------------------------------------------------------------
// Sum of the dK / dV partials of a split key block, in part order (bit-reproducible), scaled and
// rounded to the output type.  One thread per 16-byte output chunk: (tensor, b, g, key, 8 columns).
__global__ __launch_bounds__(256) void attn_bwd_dkdv_reduce_kernel(const KArgs a) {
    const int64_t rows = (int64_t)a.B * a.G * a.Skv;
    const int64_t tensor = rows * kD;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;        // chunk index over both tensors
    if (idx >= 2 * rows * 8) return;
    const int which = (int)(idx / (rows * 8));                            // 0 = dK, 1 = dV
    const int64_t rem = idx - (int64_t)which * rows * 8;
    const int64_t row = rem >> 3;
    const int c8 = (int)(rem & 7) * 8;
    const float *src = a.dkdv_partial + (int64_t)which * tensor + row * kD + c8;
    f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int part = 0; part < a.dkdv_parts; ++part) {
        const f32x4 x = *reinterpret_cast<const f32x4 *>(src + (int64_t)part * 2 * tensor);
        const f32x4 y = *reinterpret_cast<const f32x4 *>(src + (int64_t)part * 2 * tensor + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { lo[e] += x[e]; hi[e] += y[e]; }
    }
    const float mul = which == 0 ? a.scale : 1.0f;
    bf16x8 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) { out[e] = (bf16)(lo[e] * mul); out[4 + e] = (bf16)(hi[e] * mul); }
    const int key = (int)(row % a.Skv);
    const int bg = (int)(row / a.Skv);
    const int g = bg % a.G, b = bg / a.G;
    const Strides &st = which == 0 ? a.dks : a.dvs;
    bf16 *dst = (which == 0 ? a.dk : a.dv) + (int64_t)b * st.b + (int64_t)g * st.h + (int64_t)key * st.s + c8;
    union { bf16x8 v; u32x4 u; } cv;
    cv.v = out;
    *reinterpret_cast<u32x4 *>(dst) = cv.u;
}

// ---------------------------------------------------------------------------------
// dQ.  Same decomposition as the forward kernel (wavefront = 32*NQB query rows of
// one head, K/V tiles shared through LDS by HPB heads of the group):
//   S^T = K Q^T, dP^T = V dO^T, P = exp2(S*c - lse*log2e), dS = P (dP - delta),
//   dQ^T += K^T dS^T   (A = transposed read of the K tile, B = C registers).
template <bool MASKED, int NQB>
__device__ __forceinline__ void dq_tile(uint32_t ksm, uint32_t vsm, const TileLaneOffsets &lo, const bf16x8 (&qf)[NQB][4],
                                        const bf16x8 (&gf)[NQB][4], f32x16 (&dq)[NQB][2], const float (&lse2)[NQB],
                                        const float (&dlt)[NQB], const f32x16 &dseed, float c, int lane, const int (&dbase)[NQB],
                                        const unsigned (&wl)[NQB], unsigned weff, int key_lim, int wrel) {
    // wrel (masked variant only): (first query position of the wavefront) - (first key of the
    // tile); a 32-key half of the tile that no row of the wavefront can see is skipped.
    const int half = lane >> 5;
    // Masked variant, per lane and tile: key r = rc + 4*half of the tile (rc a compile-time constant per
    // accumulator register) is visible to the lane's row iff 0 <= dbase - r < wl and r < key_lim, i.e. iff
    // lo <= rc <= hi with lo = dbase - 4*half - wl + 1 and hi = min(dbase - 4*half, key_lim - 4*half - 1):
    // (unsigned)(mlo + rc) < width with mlo = -lo, width = max(0, hi - lo + 1).  One add, one compare, one
    // select per element, and no lane-dependent row index per register to keep alive across the key loop.
    // (All in wrapping 32-bit arithmetic: dbase of a dead row is about -2^30, wl at most 2^30, so the true
    // values of mlo + rc and width stay below 2^32 and 2^31.)  For 64-row wavefronts, whose register file
    // is full; the 32-row instantiations keep the plain form, which costs them no spill.
    constexpr bool FOLDED = NQB == 2;
    unsigned mlo[NQB], width[NQB];
    if (MASKED && FOLDED) {
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            const int dbh = dbase[qb] - 4 * half;
            const unsigned lo_ = (unsigned)dbh - wl[qb] + 1u;
            const int hi_ = min(dbh, key_lim - 4 * half - 1);
            mlo[qb] = 0u - lo_;
            width[qb] = (unsigned)max(0, (int)((unsigned)hi_ - lo_ + 1u));
        }
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        if (MASKED && ((32 * kb > wrel + 32 * NQB - 1) || (32 * kb + 31 < wrel - (int)weff + 1) || (32 * kb >= key_lim))) continue;
        // the dP accumulators of the first query block start at -delta (dseed, the first MFMA's C
        // operand: sixteen copies of the lane's value), so that block needs no subtraction afterwards;
        // the register file has no room for a second such block
        f32x16 s[NQB], dp[NQB];
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
            for (int i = 0; i < 16; ++i) { s[qb][i] = 0.0f; dp[qb][i] = 0.0f; }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const bf16x8 ak = ofrag_nat(ksm, lo, kb, ks);
            const bf16x8 av = ofrag_nat(vsm, lo, kb, ks);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                s[qb] = mfma_bf16(ak, qf[qb][ks], s[qb]);
                dp[qb] = mfma_bf16(av, gf[qb][ks], (ks == 0 && qb == 0) ? dseed : dp[qb]);
            }
        }
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float pe = fast_exp2(fmaf(s[qb][i], c, -lse2[qb]));
                if (MASKED && FOLDED) pe = (mlo[qb] + (unsigned)(32 * kb + 8 * (i >> 2) + (i & 3))) < width[qb] ? pe : 0.0f;
                if (MASKED && !FOLDED) {
                    const int r = 32 * kb + crow(i, half);
                    const bool vis = ((unsigned)(dbase[qb] - r) < wl[qb]) & (r < key_lim);
                    pe = vis ? pe : 0.0f;
                }
                dp[qb][i] = qb == 0 ? pe * dp[qb][i] : pe * (dp[qb][i] + dlt[qb]);        // dlt holds -delta
            }
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            bf16x8 akt[2];
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk) akt[dblk] = ofrag_tr(ksm, lo, kb, u, dblk);
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) {
                const bf16x8 dsf = cfrag(dp[qb], u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) dq[qb][dblk] = mfma_bf16(akt[dblk], dsf, dq[qb][dblk]);
            }
        }
    }
}

template <int HPB, int NQB, bool FUSE_DELTA>   // FUSE_DELTA: also produce the row statistics of the wavefront's own rows
__global__ __launch_bounds__(256, (NQB == 1 ? 3 : 2)) void attn_bwd_dq_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    constexpr int QSUB = 4 / HPB;
    constexpr int WM = 32 * NQB;
    constexpr int BM = WM * QSUB;
    constexpr int NS = 3;
    __shared__ __attribute__((aligned(16))) char smem[NS][2][kStageTileBytes];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    // For the cold paths (a tile that sticks out of the tensor, the epilogue): the wave index as a scalar and
    // the lane index recomputed on the spot, so that nothing derived from them has to survive the key loop
    // in a register file that is full (64-row wavefronts).
    const int w_s = __builtin_amdgcn_readfirstlane(w);
    auto fresh_lane = []() __attribute__((always_inline)) { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); };

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
    const int qw0 = qt * BM + WM * (w / HPB);

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window ? a.window : 0x3fffffff;

    const int bpos0 = q_offset + qt * BM;
    const int bpos1 = min(q_offset + min(a.Sq, (qt + 1) * BM) - 1, q_len - 1);
    const int hi = bpos1 >= bpos0 ? min(kv_len, bpos1 + 1) : 0;
    const int key_lo = max(0, bpos0 - weff + 1);
    const int32_t *dsrow = a.doc_start ? a.doc_start + (int64_t)b * a.Sq : nullptr;
    const int ds_b0 = dsrow ? dsrow[min(qt * BM, a.Sq - 1)] : 0;
    const int ds_w0 = dsrow ? dsrow[min(qw0, a.Sq - 1)] : 0;
    const int ds_w1 = dsrow ? dsrow[min(qw0 + WM - 1, a.Sq - 1)] : 0;
    const int t_lo = max(key_lo, ds_b0) / kTile;
    const int t_hi = hi > 0 ? (hi + kTile - 1) / kTile : 0;

    // (wave-uniform values, said so to the compiler: the tile classification then branches on scalar conditions)
    const int wpos0 = __builtin_amdgcn_readfirstlane(q_offset + qw0);
    const int wpos1 = __builtin_amdgcn_readfirstlane(min(q_offset + min(a.Sq, qw0 + WM) - 1, q_len - 1));

    const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const bf16 *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;

    bf16x8 qf[NQB][4], gf[NQB][4];
    float lse2[NQB], dlt[NQB];
    int pq[NQB];
    unsigned wl[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb) {
        const int row = qw0 + 32 * qb + l32;
        const bool row_ok = row < a.Sq;
        const bf16 *qrow = a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)row * a.qs.s;
        const bf16 *grow = a.d_o + (int64_t)b * a.dos.b + (int64_t)head * a.dos.h + (int64_t)row * a.dos.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 zq = {0u, 0u, 0u, 0u}, zg = {0u, 0u, 0u, 0u};
            if (row_ok) {
                zq = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * half);
                zg = *reinterpret_cast<const u32x4 *>(grow + 16 * ks + 8 * half);
            }
            qf[qb][ks] = as_bf16x8(zq);
            gf[qb][ks] = as_bf16x8(zg);
        }
        lse2[qb] = 0.0f;
        dlt[qb] = 0.0f;
        const int64_t off = ((int64_t)b * a.H + head) * a.Sq + row;
        if constexpr (FUSE_DELTA) {
            // No separate preprocess launch: this wavefront owns its rows, so it computes their
            // -delta = -sum_d dO*O and lse*log2(e) itself and leaves both in the scratch buffer for
            // the dK/dV and dSinks kernels, which then have to run after this one.  The lane holds
            // the 16-byte chunks 2*ks + half of its row; the sums are taken in the order of
            // attn_bwd_delta_kernel (chunk by chunk, then chunk pairs, pairs of pairs), so the
            // values are bit-identical to that kernel's.
            const bf16 *orow = a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)row * a.os.s;
            float t[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                u32x4 zo = {0u, 0u, 0u, 0u};
                if (row_ok) zo = *reinterpret_cast<const u32x4 *>(orow + 16 * ks + 8 * half);
                const bf16x8 of = as_bf16x8(zo);
                float acc = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) acc = fmaf((float)of[j], (float)gf[qb][ks][j], acc);
                t[ks] = xhalf_sum(acc);
            }
            const float dsum = (t[0] + t[1]) + (t[2] + t[3]);
            if (row_ok) {
                dlt[qb] = -dsum;
                lse2[qb] = a.lse[off] * kLog2e;
                if (half == 0 && active) {
                    a.delta[off] = dlt[qb];
                    a.delta[(int64_t)a.B * a.H * a.Sq + off] = lse2[qb];
                    a.split[off] = split_row_stats(a.lse[off], a.scale, dlt[qb]);
                }
            }
        } else if (row_ok) {
            lse2[qb] = a.delta[(int64_t)a.B * a.H * a.Sq + off];   // lse * log2(e), written by the delta kernel
            dlt[qb] = a.delta[off];                                  // -delta
        }
        const int p = q_offset + row;
        pq[qb] = (row_ok && p < q_len) ? p : -0x40000000;
        wl[qb] = (unsigned)weff;
        if (dsrow && row_ok) wl[qb] = (unsigned)min(weff, p - dsrow[row] + 1);
    }

    const float c = a.scale_log2;
    f32x16 dq[NQB][2], dseed;
#pragma unroll
    for (int i = 0; i < 16; ++i) dseed[i] = dlt[0];
#pragma unroll
    for (int qb = 0; qb < NQB; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) { dq[qb][0][i] = 0.0f; dq[qb][1][i] = 0.0f; }

    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(&smem[0][0][0]);
    const int n_it = max(0, t_hi - t_lo);
    // K / V tiles are requested in order; the pointers to the next tile's first row advance by
    // one tile per request.  Only a tile that sticks out of the tensor takes the clamping copy.
    const AsyncLaneOffsets klane = make_async_offsets(a.ks.s, lane, w), vlane = make_async_offsets(a.vs.s, lane, w);
    const bf16 *ktile = kbase + (int64_t)t_lo * kTile * a.ks.s, *vtile = vbase + (int64_t)t_lo * kTile * a.vs.s;
    int next_row0 = t_lo * kTile;
    auto issue = [&](int it) {
        const int stage = it % NS;
        if (next_row0 + kTile <= a.Skv) {
            tile_async_inner(smem[stage][0], ktile, klane, w_s);      // (scalar wave index: the LDS base is formed on the scalar unit)
            tile_async_inner(smem[stage][1], vtile, vlane, w_s);
        } else {
            const int fl = fresh_lane();
            tile_async(smem[stage][0], kbase, a.ks.s, next_row0, a.Skv, fl, w_s);
            tile_async(smem[stage][1], vbase, a.vs.s, next_row0, a.Skv, fl, w_s);
        }
        ktile += kTile * a.ks.s;
        vtile += kTile * a.vs.s;
        next_row0 += kTile;
    };
    constexpr int kLoadsPerIt = 4;

    auto iterate = [&](int it, auto stage_tag) {
        constexpr int STAGE = decltype(stage_tag)::value;
        if (it + 1 < n_it) wait_vmcnt<kLoadsPerIt>(); else wait_vmcnt<0>();
        __syncthreads();
        if (it + 2 < n_it) issue(it + 2);
        const uint32_t ksm = smem_base + STAGE * (2 * kStageTileBytes), vsm = ksm + kStageTileBytes;
        const int n0 = (t_lo + it) * kTile;
        const bool skip = !active || n0 > wpos1 || (n0 + kTile - 1) < (wpos0 - weff + 1) || wpos1 < wpos0 ||
                          (n0 + kTile - 1) < ds_w0;
        if (skip) return;
        const bool interior = (n0 + kTile - 1 <= wpos0) && (n0 > wpos1 - weff) && (n0 + kTile <= kv_len) &&
                              (q_offset + qw0 + WM - 1 <= wpos1) && (n0 >= ds_w1);
        if (interior) {
            dq_tile<false, NQB>(ksm, vsm, lo, qf, gf, dq, lse2, dlt, dseed, c, lane, pq, wl, 0u, 0, 0);
        } else {
            int dbase[NQB];
#pragma unroll
            for (int qb = 0; qb < NQB; ++qb) dbase[qb] = pq[qb] - n0;
            dq_tile<true, NQB>(ksm, vsm, lo, qf, gf, dq, lse2, dlt, dseed, c, lane, dbase, wl, (unsigned)weff, kv_len - n0, wpos0 - n0);
        }
    };

    if (n_it > 0) issue(0);
    if (n_it > 1) issue(1);
    for (int it = 0; it < n_it; it += NS) {
        iterate(it, std::integral_constant<int, 0>{});
        if (it + 1 < n_it) iterate(it + 1, std::integral_constant<int, 1>{});
        if (it + 2 < n_it) iterate(it + 2, std::integral_constant<int, 2>{});
    }
    __syncthreads();
    if (active) {
        // wave-uniform quantities recomputed from scalars
        const int hsel_s = hc * HPB + (w_s % HPB);
        const int head_s = g * a.r + hsel_s;
        const int qw0_s = qt * BM + WM * (w_s / HPB);
        const int fl = fresh_lane();
        bf16 *stage = reinterpret_cast<bf16 *>(&smem[0][0][0]) + w_s * 32 * kLS;
#pragma unroll
        for (int qb = 0; qb < NQB; ++qb) {
            const int r0 = qw0_s + 32 * qb;
            bf16 *row0 = a.dq + (int64_t)b * a.dqs.b + (int64_t)head_s * a.dqs.h + (int64_t)r0 * a.dqs.s;
            store_rows32(stage, dq[qb], a.scale, row0, a.dqs.s, a.Sq - r0, fl);
            __builtin_amdgcn_wave_barrier();
        }
    }
}

}  // namespace gptoss
