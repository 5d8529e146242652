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
#include "attn_common.h"

namespace gptoss {

// ---------------------------------------------------------------------------------
// delta[b,h,s] = sum_d dO[b,h,s,d] * O[b,h,s,d].  HBM-bound stream: eight lanes
// read one 128-byte row of each tensor, reduce with three xor-shuffles.
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(const KArgs a) {
    const int64_t rid = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3);   // (b*H + h)*Sq + s
    const int64_t total = (int64_t)a.B * a.H * a.Sq;
    if (rid >= total) return;
    const int c = threadIdx.x & 7;
    const int s = (int)(rid % a.Sq);
    const int bh = (int)(rid / a.Sq);
    const int h = bh % a.H, b = bh / a.H;
    const u32x4 ov = *reinterpret_cast<const u32x4 *>(a.o + (int64_t)b * a.os.b + (int64_t)h * a.os.h + (int64_t)s * a.os.s + c * 8);
    const u32x4 gv = *reinterpret_cast<const u32x4 *>(a.d_o + (int64_t)b * a.dos.b + (int64_t)h * a.dos.h + (int64_t)s * a.dos.s + c * 8);
    const bf16x8 of = as_bf16x8(ov), gf = as_bf16x8(gv);
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = fmaf((float)of[j], (float)gf[j], acc);
    acc += __shfl_xor(acc, 1);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 4);
    if (c == 0) a.delta[rid] = acc;
}

// ---------------------------------------------------------------------------------
// One workgroup per query head; fixed summation order, so the result is
// bit-reproducible (the reference accumulates it with relaxed atomics).
__global__ __launch_bounds__(256) void attn_bwd_dsinks_kernel(const KArgs a) {
    __shared__ float red[256];
    const int h = blockIdx.x;
    const float sink2 = (a.sinks ? a.sinks[h] : 0.0f) * kLog2e;
    float acc = 0.0f;
    for (int b = 0; b < a.B; ++b) {
        const float *lse = a.lse + ((int64_t)b * a.H + h) * a.Sq;
        const float *dl = a.delta + ((int64_t)b * a.H + h) * a.Sq;
        for (int s = threadIdx.x; s < a.Sq; s += 256)
            acc -= fast_exp2(sink2 - lse[s] * kLog2e) * dl[s];
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) a.dsinks[h] = red[0];
}

// ---------------------------------------------------------------------------------
// dK, dV.  Workgroup = 4 wavefronts x 32 keys = 128 keys of KV head g, batch b.
// K and V rows of a wavefront stay in registers as MFMA B operands.  The loop
// streams 64-row Q and dO tiles (plus their lse / delta) of each of the r query
// heads through LDS:
//   S  = Q K^T, dP = dO V^T         (A = Q / dO rows from LDS, natural reads)
//   P  = exp2(S*c - lse*log2e),  dS = P * (dP - delta)
//   dV^T += dO^T P,  dK^T += Q^T dS (A = transposed LDS reads, B = C registers)
// A lane owns one key; accumulators are written once at the end.
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(const KArgs a) {
    constexpr int BN = 128;
    __shared__ __attribute__((aligned(16))) bf16 smem[2][2][kTileElems];
    __shared__ __attribute__((aligned(16))) float sstat[2][2][kTile];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;

    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int b = bid % a.B; bid /= a.B;
    const int kt = bid;                                   // ascending: most work first
    const int j0 = kt * BN;                               // first key of the workgroup
    const int wj0 = j0 + 32 * w;                          // first key of the wavefront
    const int jme = wj0 + l32;                            // this lane's key

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window ? a.window : 0x3fffffff;

    // query rows that can see any key of the workgroup
    const int j1 = min(j0 + BN, kv_len) - 1;              // last live key
    int i_lo = max(0, j0 - a.q_offset);
    int64_t i_hi64 = min((int64_t)a.Sq, (int64_t)q_len - a.q_offset);
    i_hi64 = min(i_hi64, (int64_t)j1 + weff - a.q_offset);
    const int i_hi = (j1 >= j0) ? (int)max((int64_t)0, i_hi64) : 0;
    const int qt_lo = i_lo / kTile;
    const int qt_hi = (i_hi + kTile - 1) / kTile;
    const int nq = max(0, qt_hi - qt_lo);
    const int n_it = nq * a.r;

    // K, V fragments (B operands): lane = key, slots = head_dim
    bf16x8 kf[4], vf[4];
    {
        const bf16 *krow = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h + (int64_t)jme * a.ks.s;
        const bf16 *vrow = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h + (int64_t)jme * a.vs.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 zk = {0u, 0u, 0u, 0u}, zv = {0u, 0u, 0u, 0u};
            if (jme < a.Skv) {
                zk = *reinterpret_cast<const u32x4 *>(krow + 16 * ks + 8 * half);
                zv = *reinterpret_cast<const u32x4 *>(vrow + 16 * ks + 8 * half);
            }
            kf[ks] = as_bf16x8(zk);
            vf[ks] = as_bf16x8(zv);
        }
    }

    f32x16 dk[2], dv[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk[0][i] = dk[1][i] = 0.0f; dv[0][i] = dv[1][i] = 0.0f; }

    const float c = a.scale_log2;
    TileRegs qr, gr;
    float st = 0.0f;     // lse*log2e (threads 0..63) or delta (threads 64..127) of the staged tile

    auto prefetch = [&](int it) {
        const int hq = g * a.r + it / nq;
        const int i0 = (qt_lo + it % nq) * kTile;
        tile_load(qr, a.q + (int64_t)b * a.qs.b + (int64_t)hq * a.qs.h, a.qs.s, i0, a.Sq, tid);
        tile_load(gr, a.d_o + (int64_t)b * a.dos.b + (int64_t)hq * a.dos.h, a.dos.s, i0, a.Sq, tid);
        if (tid < 128) {
            const int i = i0 + (tid & 63);
            const int64_t off = ((int64_t)b * a.H + hq) * a.Sq + i;
            st = 0.0f;
            if (i < a.Sq) st = (tid < 64) ? a.lse[off] * kLog2e : a.delta[off];
        }
    };

    if (n_it > 0) prefetch(0);
    for (int it = 0; it < n_it; ++it) {
        const int buf = it & 1;
        bf16 *qsm = smem[buf][0], *gsm = smem[buf][1];
        tile_store(qsm, qr, tid);
        tile_store(gsm, gr, tid);
        if (tid < 128) sstat[buf][tid >> 6][tid & 63] = st;
        __syncthreads();
        if (it + 1 < n_it) prefetch(it + 1);

        const int i0 = (qt_lo + it % nq) * kTile;
        const int pos0 = a.q_offset + i0;                                    // first query position of the tile
        const int pos1 = min(a.q_offset + min(a.Sq, i0 + kTile) - 1, q_len - 1);   // last live one
        const int wj1 = min(wj0 + 32, kv_len) - 1;                           // wavefront's last live key
        const bool skip = wj1 < wj0 || pos1 < wj0 || pos0 > wj1 + weff - 1 || pos1 < pos0;
        if (skip) continue;
        const bool interior = (wj0 + 31 <= pos0) && (wj0 > pos1 - weff) && (wj0 + 32 <= kv_len) &&
                              (a.q_offset + i0 + kTile - 1 <= pos1);
        const float *lse_s = sstat[buf][0], *del_s = sstat[buf][1];

#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            f32x16 s, dp;
#pragma unroll
            for (int i = 0; i < 16; ++i) { s[i] = 0.0f; dp[i] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                s = mfma_bf16(frag_nat(qsm, qb, ks, lane), kf[ks], s);
                dp = mfma_bf16(frag_nat(gsm, qb, ks, lane), vf[ks], dp);
            }
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const f32x4 lv = *reinterpret_cast<const f32x4 *>(lse_s + 32 * qb + 8 * a4 + 4 * half);
                const f32x4 dl = *reinterpret_cast<const f32x4 *>(del_s + 32 * qb + 8 * a4 + 4 * half);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = 4 * a4 + e;
                    float pe = fast_exp2(fmaf(s[i], c, -lv[e]));
                    if (!interior) {
                        const int irow = i0 + 32 * qb + 8 * a4 + 4 * half + e;
                        const int p = a.q_offset + irow;
                        const bool vis = (irow < a.Sq) && (p < q_len) && (jme <= p) && (jme > p - weff) && (jme < kv_len);
                        pe = vis ? pe : 0.0f;
                    }
                    s[i] = pe;
                    dp[i] = pe * (dp[i] - dl[e]);
                }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const bf16x8 pf = cfrag(s, u), dsf = cfrag(dp, u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) {
                    dv[dblk] = mfma_bf16(frag_tr(gsm, qb, u, dblk, lane), pf, dv[dblk]);
                    dk[dblk] = mfma_bf16(frag_tr(qsm, qb, u, dblk, lane), dsf, dk[dblk]);
                }
            }
        }
    }

    __syncthreads();
    bf16 *stage = &smem[0][0][0] + w * 32 * kLS;
    const int nvalid = a.Skv - wj0;
    store_rows32(stage, dk, a.scale, a.dk + (int64_t)b * a.dks.b + (int64_t)g * a.dks.h + (int64_t)wj0 * a.dks.s,
                 a.dks.s, nvalid, lane);
    __builtin_amdgcn_wave_barrier();
    store_rows32(stage, dv, 1.0f, a.dv + (int64_t)b * a.dvs.b + (int64_t)g * a.dvs.h + (int64_t)wj0 * a.dvs.s,
                 a.dvs.s, nvalid, lane);
}

// ---------------------------------------------------------------------------------
// dQ.  Same decomposition as the forward kernel (wavefront = 32 query rows of one
// head, K/V tiles shared through LDS by HPB heads of the group):
//   S^T = K Q^T, dP^T = V dO^T, P = exp2(S*c - lse*log2e), dS = P (dP - delta),
//   dQ^T += K^T dS^T   (A = transposed read of the K tile, B = C registers).
template <int HPB>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(const KArgs a) {
    constexpr int QSUB = 4 / HPB;
    constexpr int BM = 32 * QSUB;
    __shared__ __attribute__((aligned(16))) bf16 smem[2][2][kTileElems];

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;

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
    const int qw0 = qt * BM + 32 * (w / HPB);

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window ? a.window : 0x3fffffff;

    const int bpos0 = a.q_offset + qt * BM;
    const int bpos1 = min(a.q_offset + min(a.Sq, (qt + 1) * BM) - 1, q_len - 1);
    const int hi = bpos1 >= bpos0 ? min(kv_len, bpos1 + 1) : 0;
    const int lo = max(0, bpos0 - weff + 1);
    const int t_lo = lo / kTile;
    const int t_hi = hi > 0 ? (hi + kTile - 1) / kTile : 0;

    const int wpos0 = a.q_offset + qw0;
    const int wpos1 = min(a.q_offset + min(a.Sq, qw0 + 32) - 1, q_len - 1);
    const int p = wpos0 + l32;
    const bool row_ok = qw0 + l32 < a.Sq;
    const bool p_ok = row_ok && (p < q_len);

    const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const bf16 *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;

    bf16x8 qf[4], gf[4];
    {
        const bf16 *qrow = a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)(qw0 + l32) * a.qs.s;
        const bf16 *grow = a.d_o + (int64_t)b * a.dos.b + (int64_t)head * a.dos.h + (int64_t)(qw0 + l32) * a.dos.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 zq = {0u, 0u, 0u, 0u}, zg = {0u, 0u, 0u, 0u};
            if (row_ok) {
                zq = *reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * half);
                zg = *reinterpret_cast<const u32x4 *>(grow + 16 * ks + 8 * half);
            }
            qf[ks] = as_bf16x8(zq);
            gf[ks] = as_bf16x8(zg);
        }
    }
    float lse2 = 0.0f, dlt = 0.0f;
    if (row_ok) {
        const int64_t off = ((int64_t)b * a.H + head) * a.Sq + qw0 + l32;
        lse2 = a.lse[off] * kLog2e;
        dlt = a.delta[off];
    }

    const float c = a.scale_log2;
    f32x16 dq[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { dq[0][i] = 0.0f; dq[1][i] = 0.0f; }

    TileRegs kr, vr;
    if (t_lo < t_hi) {
        tile_load(kr, kbase, a.ks.s, t_lo * kTile, a.Skv, tid);
        tile_load(vr, vbase, a.vs.s, t_lo * kTile, a.Skv, tid);
    }
    for (int t = t_lo; t < t_hi; ++t) {
        const int buf = (t - t_lo) & 1;
        bf16 *ksm = smem[buf][0], *vsm = smem[buf][1];
        tile_store(ksm, kr, tid);
        tile_store(vsm, vr, tid);
        __syncthreads();
        if (t + 1 < t_hi) {
            tile_load(kr, kbase, a.ks.s, (t + 1) * kTile, a.Skv, tid);
            tile_load(vr, vbase, a.vs.s, (t + 1) * kTile, a.Skv, tid);
        }
        const int n0 = t * kTile;
        const bool skip = !active || n0 > wpos1 || (n0 + kTile - 1) < (wpos0 - weff + 1) || wpos1 < wpos0;
        if (skip) continue;
        const bool interior = (n0 + kTile - 1 <= wpos0) && (n0 > wpos1 - weff) && (n0 + kTile <= kv_len) &&
                              (a.q_offset + qw0 + 31 <= wpos1);
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            f32x16 s, dp;
#pragma unroll
            for (int i = 0; i < 16; ++i) { s[i] = 0.0f; dp[i] = 0.0f; }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                s = mfma_bf16(frag_nat(ksm, blk, ks, lane), qf[ks], s);
                dp = mfma_bf16(frag_nat(vsm, blk, ks, lane), gf[ks], dp);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float pe = fast_exp2(fmaf(s[i], c, -lse2));
                if (!interior) {
                    const int j = n0 + 32 * blk + crow(i, half);
                    const bool vis = p_ok && (j <= p) && (j > p - weff) && (j < kv_len);
                    pe = vis ? pe : 0.0f;
                }
                dp[i] = pe * (dp[i] - dlt);
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const bf16x8 dsf = cfrag(dp, u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk)
                    dq[dblk] = mfma_bf16(frag_tr(ksm, blk, u, dblk, lane), dsf, dq[dblk]);
            }
        }
    }
    __syncthreads();
    if (active) {
        bf16 *stage = &smem[0][0][0] + w * 32 * kLS;
        bf16 *row0 = a.dq + (int64_t)b * a.dqs.b + (int64_t)head * a.dqs.h + (int64_t)qw0 * a.dqs.s;
        store_rows32(stage, dq, a.scale, row0, a.dqs.s, a.Sq - qw0, lane);
    }
}

}  // namespace gptoss
