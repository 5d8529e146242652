// float32 kernels (dtype GPTOSS_ATTN_FP32): the same forward / backward as the bf16 kernels
// for callers that keep the model in float32 (the reference runs such tensors natively,
// attention_kernel.py:11-217 are dtype-generic).  They exist for exactness, not speed: every
// product runs on the fp32 matrix instruction v_mfma_f32_32x32x2_f32 with fp32 operands
// straight from global memory (the L1/L2 caches do the sharing; there is no LDS staging), and
// every element evaluates the full visibility predicate.
//
// One wavefront is independent of every other (no LDS, no barrier):
//   forward, dQ : a wavefront owns 32 query rows of one head and walks 32-key tiles;
//   dK/dV       : a wavefront owns 32 keys of one KV head and walks the query heads of the
//                 group and their 32-row blocks.
// Register layouts of v_mfma_f32_32x32x2_f32 (lane = 0..63, half = lane/32, l32 = lane%32):
//   A (32 x 2): lane holds A[l32][half]      B (2 x 32): lane holds B[half][l32]
//   C (32 x 32): register i holds C[crow(i, half)][l32]   (as for the bf16 instruction)
// A contraction over head_dim takes 32 such steps; step ks uses d = 32*half + ks, so a lane
// reads 32 CONSECUTIVE floats of its row.  A contraction over the 32 rows held in C registers
// takes 16 steps: step (a4, e) multiplies C register 4*a4 + e, whose row is 8*a4 + 4*half + e,
// by the matching row of the other operand -- C registers are fed back as the B operand
// without any data movement.
#pragma once
#include "attn_common.h"

namespace gptoss {

__device__ __forceinline__ f32x16 mfma_f32(float a, float b, const f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

struct F32Ptrs {
    const float *q, *k, *v, *d_o;
    float *o, *dq, *dk, *dv;
};
__device__ __forceinline__ F32Ptrs f32_ptrs(const KArgs &a) {
    F32Ptrs p;
    p.q = reinterpret_cast<const float *>(a.q);
    p.k = reinterpret_cast<const float *>(a.k);
    p.v = reinterpret_cast<const float *>(a.v);
    p.d_o = reinterpret_cast<const float *>(a.d_o);
    p.o = reinterpret_cast<float *>(a.o);
    p.dq = reinterpret_cast<float *>(a.dq);
    p.dk = reinterpret_cast<float *>(a.dk);
    p.dv = reinterpret_cast<float *>(a.dv);
    return p;
}

// 32 consecutive floats starting at p (16-byte aligned) into r[0..31]; zero when !valid.
__device__ __forceinline__ void load_row32(float (&r)[32], const float *p, bool valid) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        if (valid) z = *reinterpret_cast<const f32x4 *>(p + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; ++e) r[4 * j + e] = z[e];
    }
}

// Per-lane description of one query row.
struct RowInfo {
    int pos;        // absolute position, hugely negative for a row that does not exist / is padding
    unsigned win;   // visible keys are pos - win < key <= pos
};
__device__ __forceinline__ RowInfo row_info(const KArgs &a, int q_offset, int b, int row, int q_len) {
    RowInfo r;
    const int p = q_offset + row;
    const bool live = row < a.Sq && p < q_len;
    r.pos = live ? p : -0x40000000;
    int w = a.window ? a.window : 0x3fffffff;
    if (a.doc_start && row < a.Sq) w = min(w, p - a.doc_start[(int64_t)b * a.Sq + row] + 1);
    r.win = (unsigned)w;
    return r;
}
__device__ __forceinline__ bool visible(const RowInfo &r, int key, int kv_len) {
    return ((unsigned)(r.pos - key) < r.win) & (key < kv_len);
}

// wavefront index -> (batch, head-like index, 32-row block); false when out of range
__device__ __forceinline__ bool wave_work(int n_blk, int n_head, int n_batch, int &b, int &h, int &blk) {
    const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wid >= (int64_t)n_blk * n_head * n_batch) return false;
    blk = (int)(wid % n_blk);
    h = (int)((wid / n_blk) % n_head);
    b = (int)(wid / ((int64_t)n_blk * n_head));
    return true;
}

// ---- forward ------------------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_f32_fwd_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    const F32Ptrs t = f32_ptrs(a);
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5;
    int b, head, qblk;
    if (!wave_work((a.Sq + 31) / 32, a.H, a.B, b, head, qblk)) return;
    const int g = head / a.r;
    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int q0 = 32 * qblk, row = q0 + l32;
    const RowInfo ri = row_info(a, q_offset, b, row, q_len);

    float qr[32];    // Q[row][32*half + ks]
    load_row32(qr, t.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)min(row, a.Sq - 1) * a.qs.s + 32 * half, row < a.Sq);
    const float *kb = t.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const float *vb = t.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;

    const float c = a.scale_log2;
    const float sink2 = (a.sinks ? a.sinks[head] : 0.0f) * kLog2e;
    float m = sink2, l = 0.0f;
    f32x16 o[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { o[0][i] = 0.0f; o[1][i] = 0.0f; }

    // keys any row of this block can see: [key_lo, key_hi)
    const int weff = a.window ? a.window : 0x3fffffff;
    const int pos_hi = min(q_offset + min(a.Sq, q0 + 32) - 1, q_len - 1);
    const int key_hi = pos_hi >= q_offset + q0 ? min(kv_len, pos_hi + 1) : 0;
    const int key_lo = max(0, q_offset + q0 - weff + 1);
    for (int n0 = (key_lo / 32) * 32; n0 < key_hi; n0 += 32) {
        float kr[32];    // K[n0 + l32][32*half + ks]
        load_row32(kr, kb + (int64_t)min(n0 + l32, a.Skv - 1) * a.ks.s + 32 * half, true);
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 32; ++ks) s = mfma_f32(kr[ks], qr[ks], s);      // S^T: rows = keys, lane = query row
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = visible(ri, n0 + crow(i, half), kv_len) ? s[i] * c : -INFINITY;
            mx = fmaxf(mx, s[i]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m, mx);
        const float alpha = exp2f(m - m_new);
        m = m_new;
        l *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) { o[0][i] *= alpha; o[1][i] *= alpha; }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = exp2f(s[i] - m);
            l += s[i];
        }
        // O^T[d][row] += V^T[d][key] P^T[key][row]
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float *vrow = vb + (int64_t)min(n0 + 8 * a4 + 4 * half + e, a.Skv - 1) * a.vs.s;
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) o[dblk] = mfma_f32(vrow[32 * dblk + l32], s[4 * a4 + e], o[dblk]);
            }
    }

    const float l_tot = l + __shfl_xor(l, 32);
    const float z = l_tot + exp2f(sink2 - m);
    const float inv = 1.0f / z;
    if (row < a.Sq) {
        float *orow = t.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)row * a.os.s;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                f32x4 w4;
#pragma unroll
                for (int e = 0; e < 4; ++e) w4[e] = o[dblk][4 * a4 + e] * inv;
                *reinterpret_cast<f32x4 *>(orow + 32 * dblk + 8 * a4 + 4 * half) = w4;
            }
        if (half == 0) a.lse[((int64_t)b * a.H + head) * a.Sq + row] = (m + log2f(z)) * kLn2;
    }
}

// ---- backward step 1: -delta and lse*log2(e) into the scratch (same layout as the bf16 path) ----
__global__ __launch_bounds__(256) void attn_f32_delta_kernel(const KArgs a) {
    const F32Ptrs t = f32_ptrs(a);
    const int64_t total = (int64_t)a.B * a.H * a.Sq;
    const int c = threadIdx.x & 15;                                   // 16 lanes x 16 bytes = one 256-byte row
    const int64_t rid = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    float acc = 0.0f;
    if (rid < total) {
        const int s = (int)(rid % a.Sq);
        const int bh = (int)(rid / a.Sq);
        const int h = bh % a.H, b = bh / a.H;
        const f32x4 ov = *reinterpret_cast<const f32x4 *>(t.o + (int64_t)b * a.os.b + (int64_t)h * a.os.h + (int64_t)s * a.os.s + 4 * c);
        const f32x4 gv = *reinterpret_cast<const f32x4 *>(t.d_o + (int64_t)b * a.dos.b + (int64_t)h * a.dos.h + (int64_t)s * a.dos.s + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = fmaf(ov[e], gv[e], acc);
    }
    acc += __shfl_xor(acc, 1);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 4);
    acc += __shfl_xor(acc, 8);
    if (c == 0 && rid < total) {
        a.delta[rid] = -acc;
        a.delta[total + rid] = a.lse[rid] * kLog2e;
    }
}

// ---- backward step 2: dK, dV ------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_f32_dkdv_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    const F32Ptrs t = f32_ptrs(a);
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5;
    int b, g, kblk;
    if (!wave_work((a.Skv + 31) / 32, a.G, a.B, b, g, kblk)) return;
    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int j0 = 32 * kblk, key = j0 + l32;
    const int64_t total = (int64_t)a.B * a.H * a.Sq;

    float kr[32], vr[32];    // K / V[key][32*half + ks]  (B operands of S and dP)
    load_row32(kr, t.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h + (int64_t)min(key, a.Skv - 1) * a.ks.s + 32 * half, key < a.Skv);
    load_row32(vr, t.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h + (int64_t)min(key, a.Skv - 1) * a.vs.s + 32 * half, key < a.Skv);
    f32x16 dk[2], dv[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk[0][i] = dk[1][i] = 0.0f; dv[0][i] = dv[1][i] = 0.0f; }

    // query rows that can see any key of the block: positions [j0, j0 + 31 + window)
    const int weff = a.window ? a.window : 0x3fffffff;
    const int row_lo = max(0, j0 - q_offset);
    const int64_t row_hi64 = min((int64_t)min(a.Sq, max(0, q_len - q_offset)), (int64_t)j0 + 31 + weff - q_offset);
    const int row_hi = j0 < kv_len ? (int)row_hi64 : 0;
    const float c = a.scale_log2;
    for (int hh = 0; hh < a.r; ++hh) {
        const int head = g * a.r + hh;
        const float *qb = t.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h;
        const float *gb = t.d_o + (int64_t)b * a.dos.b + (int64_t)head * a.dos.h;
        const float *nd = a.delta + ((int64_t)b * a.H + head) * a.Sq;     // -delta
        const float *l2 = nd + total;                                      // lse * log2(e)
        for (int q0 = (row_lo / 32) * 32; q0 < row_hi; q0 += 32) {
            const int qrow = min(q0 + l32, a.Sq - 1);
            float qr[32], gr[32];   // Q / dO[q0 + l32][32*half + ks]  (A operands)
            load_row32(qr, qb + (int64_t)qrow * a.qs.s + 32 * half, true);
            load_row32(gr, gb + (int64_t)qrow * a.dos.s + 32 * half, true);
            f32x16 s, dp;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                s[i] = 0.0f;
                dp[i] = nd[min(q0 + crow(i, half), a.Sq - 1)];          // seeds dP with -delta of its row
            }
#pragma unroll
            for (int ks = 0; ks < 32; ++ks) {
                s = mfma_f32(qr[ks], kr[ks], s);                          // rows = queries, lane = key
                dp = mfma_f32(gr[ks], vr[ks], dp);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = q0 + crow(i, half);
                RowInfo ri = row_info(a, q_offset, b, row, q_len);
                const float p = visible(ri, key, kv_len) ? exp2f(fmaf(s[i], c, -l2[min(row, a.Sq - 1)])) : 0.0f;
                s[i] = p;
                dp[i] = p * dp[i];                                        // dS (without the softmax scale)
            }
            // dV^T[d][key] += dO^T[d][row] P[row][key];  dK^T[d][key] += Q^T[d][row] dS[row][key]
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = min(q0 + 8 * a4 + 4 * half + e, a.Sq - 1);
                    const float *grow = gb + (int64_t)r * a.dos.s;
                    const float *qrow2 = qb + (int64_t)r * a.qs.s;
#pragma unroll
                    for (int dblk = 0; dblk < 2; ++dblk) {
                        dv[dblk] = mfma_f32(grow[32 * dblk + l32], s[4 * a4 + e], dv[dblk]);
                        dk[dblk] = mfma_f32(qrow2[32 * dblk + l32], dp[4 * a4 + e], dk[dblk]);
                    }
                }
        }
    }
    if (key < a.Skv) {
        float *dkrow = t.dk + (int64_t)b * a.dks.b + (int64_t)g * a.dks.h + (int64_t)key * a.dks.s;
        float *dvrow = t.dv + (int64_t)b * a.dvs.b + (int64_t)g * a.dvs.h + (int64_t)key * a.dvs.s;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                f32x4 wk, wv;
#pragma unroll
                for (int e = 0; e < 4; ++e) { wk[e] = dk[dblk][4 * a4 + e] * a.scale; wv[e] = dv[dblk][4 * a4 + e]; }
                *reinterpret_cast<f32x4 *>(dkrow + 32 * dblk + 8 * a4 + 4 * half) = wk;
                *reinterpret_cast<f32x4 *>(dvrow + 32 * dblk + 8 * a4 + 4 * half) = wv;
            }
    }
}

// ---- backward step 3: dQ ----------------------------------------------------------------
__global__ __launch_bounds__(256) void attn_f32_dq_kernel(const KArgs a) {
    const int q_offset = query_offset(a);
    const F32Ptrs t = f32_ptrs(a);
    const int lane = threadIdx.x & 63, l32 = lane & 31, half = lane >> 5;
    int b, head, qblk;
    if (!wave_work((a.Sq + 31) / 32, a.H, a.B, b, head, qblk)) return;
    const int g = head / a.r;
    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int q0 = 32 * qblk, row = q0 + l32;
    const RowInfo ri = row_info(a, q_offset, b, row, q_len);
    const int64_t total = (int64_t)a.B * a.H * a.Sq;
    const int rowc = min(row, a.Sq - 1);

    float qr[32], gr[32];
    load_row32(qr, t.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)rowc * a.qs.s + 32 * half, row < a.Sq);
    load_row32(gr, t.d_o + (int64_t)b * a.dos.b + (int64_t)head * a.dos.h + (int64_t)rowc * a.dos.s + 32 * half, row < a.Sq);
    const float ndelta = a.delta[((int64_t)b * a.H + head) * a.Sq + rowc];
    const float lse2 = a.delta[total + ((int64_t)b * a.H + head) * a.Sq + rowc];
    const float *kb = t.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const float *vb = t.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;
    const float c = a.scale_log2;
    f32x16 dq[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) { dq[0][i] = 0.0f; dq[1][i] = 0.0f; }

    const int weff = a.window ? a.window : 0x3fffffff;
    const int pos_hi = min(q_offset + min(a.Sq, q0 + 32) - 1, q_len - 1);
    const int key_hi = pos_hi >= q_offset + q0 ? min(kv_len, pos_hi + 1) : 0;
    const int key_lo = max(0, q_offset + q0 - weff + 1);
    for (int n0 = (key_lo / 32) * 32; n0 < key_hi; n0 += 32) {
        const int krow = min(n0 + l32, a.Skv - 1);
        float kr[32], vr[32];
        load_row32(kr, kb + (int64_t)krow * a.ks.s + 32 * half, true);
        load_row32(vr, vb + (int64_t)krow * a.vs.s + 32 * half, true);
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) { s[i] = 0.0f; dp[i] = ndelta; }
#pragma unroll
        for (int ks = 0; ks < 32; ++ks) {
            s = mfma_f32(kr[ks], qr[ks], s);          // S^T
            dp = mfma_f32(vr[ks], gr[ks], dp);        // dP^T - delta
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = visible(ri, n0 + crow(i, half), kv_len) ? exp2f(fmaf(s[i], c, -lse2)) : 0.0f;
            dp[i] = p * dp[i];
        }
        // dQ^T[d][row] += K^T[d][key] dS^T[key][row]
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float *krow2 = kb + (int64_t)min(n0 + 8 * a4 + 4 * half + e, a.Skv - 1) * a.ks.s;
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk) dq[dblk] = mfma_f32(krow2[32 * dblk + l32], dp[4 * a4 + e], dq[dblk]);
            }
    }
    if (row < a.Sq) {
        float *dqrow = t.dq + (int64_t)b * a.dqs.b + (int64_t)head * a.dqs.h + (int64_t)row * a.dqs.s;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                f32x4 w4;
#pragma unroll
                for (int e = 0; e < 4; ++e) w4[e] = dq[dblk][4 * a4 + e] * a.scale;
                *reinterpret_cast<f32x4 *>(dqrow + 32 * dblk + 8 * a4 + 4 * half) = w4;
            }
    }
}

}  // namespace gptoss
