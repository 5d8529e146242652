// Forward kernel for sliding-window layers whose window is 32, 64, 96 or 128 keys: the same results as
// attn_fwd_kernel (the reference's `_attn_fwd`, attention_kernel.py:11-100, with `bandwidth` set), computed with
// a softmax that is not "online".
//
// Why.  A 32-row query block of such a layer sees window + 32 keys, which is few enough to hold every logit of
// the block in registers at once (16 per 32-key block and lane).  The row maximum is then known before the first
// exponential: no running maximum, no rescaling of the accumulator from tile to tile, one exchange between the
// lane halves instead of one per tile, no tile classification, no loop.  attn_fwd_kernel spends about 1040 vector
// instructions per wavefront on such a block against 40 MFMAs and is bound by the issue of those; this kernel
// needs about half.
//
// Work split.  As in attn_fwd_kernel with 32-row wavefronts: a workgroup is four query heads of one KV head on
// the same 32 query rows r0 .. r0 + 31, so the keys r0 - W .. r0 + 31 (W + 32 rows of K and of V) are staged in
// LDS once for the four of them, in one go.
//
// Masks.  With W a multiple of 32 the key range is NH = W / 32 + 1 blocks of 32 keys.  The blocks in the middle
// are visible to every row.  Row i of the wavefront sees key j of the first block iff j > i and key j of the last
// block iff j <= i: the two masks are complementary, so the kernel merges the two blocks' logits into ONE block
// (16 selects per lane), runs maximum, exponential and row sum on that, and takes it apart again (with zeros)
// only as the bf16 operand of the second GEMM.  Query blocks whose window would start before key 0 (the first
// W / 32 blocks of a row) take a plain variant with a general test on every element.
#pragma once
#include <type_traits>

#include "attn_common.h"

namespace gptoss {

template <int WH>
struct FwdWindow {
    static constexpr int W = 32 * WH;              // window, in keys
    static constexpr int NH = WH + 1;              // 32-key blocks a 32-row query block can see
    static constexpr int kRows = 32 * NH;          // rows of K (and of V) staged per workgroup
    static constexpr int kTileBytes = kRows * kRowBytes;
    static constexpr int kStageBytes = 4 * 32 * kLS * 2;             // the four wavefronts' output rows pass through the K buffer
    static constexpr int kKBytes = kTileBytes > kStageBytes ? kTileBytes : kStageBytes;
};

// max(a, b, c): the compiler makes one v_max3_f32 of it where it knows the operands to be results of arithmetic (no
// signalling NaN to quiet), which is the case for everything it is used on here.  Not inline assembly: the wait states
// between an MFMA and a vector instruction that reads its result are the compiler's to insert, and it does not look
// into assembly text.
__device__ __forceinline__ float max3_f32(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }

template <int WH>
__global__ __launch_bounds__(256, 3) void attn_fwd_window_kernel(const KArgs a) {
    using C = FwdWindow<WH>;
    constexpr int W = C::W, NH = C::NH;
    __shared__ __attribute__((aligned(16))) char smem[C::kKBytes + C::kTileBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;

    // workgroup (x, y, z) = (kv head, batch row and group of four query heads, 32-row query block); workgroups are dealt
    // to the XCDs in x-fastest order, so that with G == 8 each XCD keeps one KV head's K / V in its own L2
    const int n_hc = a.r >> 2;
    const int g = blockIdx.x;
    const int b = blockIdx.y / n_hc, hc = blockIdx.y - b * n_hc;
    const int r0 = 32 * blockIdx.z;                // first query row of the workgroup
    const int head = g * a.r + 4 * hc + w;
    const int k0 = r0 - W;                         // first staged key; negative for the first WH blocks of a row
    const bool edge = k0 < 0;
    // right-padded batch rows: query rows at or beyond the row's length have no keys (O = 0, lse = the sink logit); the
    // rows that exist never see a key beyond it
    const int len = a.seqlens ? min(max(a.seqlens[b], 0), a.Sq) : a.Sq;
    if (r0 >= len) {
        // nothing but padding in this block
        const float sink_lse = ((a.sinks ? a.sinks[head] : 0.0f) * kLog2e + fast_log2(1.0f)) * kLn2;   // what the epilogue below gives a row without keys
        bf16 *orow = a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)(r0 + (lane >> 3)) * a.os.s + (lane & 7) * 8;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) *reinterpret_cast<u32x4 *>(orow + (int64_t)(8 * pass) * a.os.s) = u32x4{0u, 0u, 0u, 0u};
        if (half == 0) a.lse[((int64_t)b * a.H + head) * a.Sq + r0 + l32] = sink_lse;
        return;
    }
    const bool no_keys = r0 + l32 >= len;          // this lane's row is padding

    bf16x8 qf[4];                                  // Q^T fragments (B operand)
    {
        const char *qblk = reinterpret_cast<const char *>(a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)r0 * a.qs.s);
        const uint32_t qoff = (uint32_t)(l32 * (int)a.qs.s + 8 * half) * 2u;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qf[ks] = as_bf16x8(*reinterpret_cast<const u32x4 *>(qblk + qoff + 32 * ks));
    }
    const uint32_t ksm = lds_addr(smem), vsm = ksm + C::kKBytes;
    {
        // copy j of wavefront w fills rows 8 (w + 4 j) .. + 7 of the staged range; rows in front of key 0 re-read key 0
        // (their logits are masked, they only have to be finite)
        const int rloc = 8 * w + (lane >> 3);
        const int ch = (lane & 7) ^ swz(rloc);     // swz() of the row: 32 j does not reach the bits it looks at
        const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h, *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;
        char *kdst = smem + w * 8 * kRowBytes, *vdst = smem + C::kKBytes + w * 8 * kRowBytes;
        // addresses are (scalar pointer) + (32-bit lane offset): the row of copy j is a scalar step away from copy 0's,
        // except where rows are held at key 0
        auto copy_all = [&](const bf16 *base, int stride, char *dst) __attribute__((always_inline)) {
            if (!edge) {
                const uint32_t voff = (uint32_t)(rloc * stride + ch * 8) * 2u;
#pragma unroll
                for (int j = 0; j < NH; ++j)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(reinterpret_cast<const char *>(base + (int64_t)(k0 + 32 * j) * stride) + voff),
                                                     (lds_void_t *)(dst + j * 32 * kRowBytes), 16, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < NH; ++j) {
                    const uint32_t voff = (uint32_t)(max(k0 + rloc + 32 * j, 0) * stride + ch * 8) * 2u;
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(reinterpret_cast<const char *>(base) + voff),
                                                     (lds_void_t *)(dst + j * 32 * kRowBytes), 16, 0, 0);
                }
            }
        };
        copy_all(kbase, (int)a.ks.s, kdst);
        copy_all(vbase, (int)a.vs.s, vdst);
    }

    const float c = a.scale_log2;
    const float sink2 = (a.sinks ? a.sinks[head] : 0.0f) * kLog2e;
    const TileLaneOffsets lo = make_tile_offsets(lane);
    const int x = l32 - 4 * half;                  // register i of a block holds key rc(i) + 4 half: "key <= row" is rc(i) <= x

    wait_vmcnt<0>();                               // this wavefront's copies of K and V (and its Q rows) have landed ...
    __syncthreads();                               // ... and everybody else's

    // S^T = K Q^T for all NH blocks: lane = query row l32, register i of block h = key 32 h + rc(i) + 4 half
    f32x16 s[NH];
    const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        s[h] = mfma_bf16(ofrag_nat(ksm, lo, h, 0), qf[0], zero16);
#pragma unroll
        for (int ks = 1; ks < 4; ++ks) s[h] = mfma_bf16(ofrag_nat(ksm, lo, h, ks), qf[ks], s[h]);
    }

    f32x16 o[2];
    float m, l;
    if (!edge) {
        // the first and the last block as one: register i is the last block's key where the row may see it, else the
        // first block's
        f32x16 &t = s[0];
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = (8 * (i >> 2) + (i & 3) <= x) ? s[NH - 1][i] : t[i];
        float mx0 = max3_f32(t[0], t[1], t[2]), mx1 = max3_f32(t[3], t[4], t[5]);
#pragma unroll
        for (int i = 6; i < 14; i += 4) { mx0 = max3_f32(mx0, t[i], t[i + 1]); mx1 = max3_f32(mx1, t[i + 2], t[i + 3]); }
        mx0 = max3_f32(mx0, t[14], t[15]);
#pragma unroll
        for (int h = 1; h < NH - 1; ++h)
#pragma unroll
            for (int i = 0; i < 16; i += 4) { mx0 = max3_f32(mx0, s[h][i], s[h][i + 1]); mx1 = max3_f32(mx1, s[h][i + 2], s[h][i + 3]); }
        m = fast_max(sink2, xhalf_max(fast_max(mx0, mx1)) * c);       // the reference starts its maximum at the sink logit (ref :53)
        m = no_keys ? sink2 : m;
        const float nm = no_keys ? -INFINITY : -m;                     // a row of padding: every weight exp2(-inf) = 0

        float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float e0 = fast_exp2(fmaf(t[i], c, nm)), e1 = fast_exp2(fmaf(t[i + 1], c, nm));
            t[i] = e0; t[i + 1] = e1;
            rs0 += e0; rs1 += e1;
        }
        // the merged block taken apart: what a row sees of the first block, and of the last
        f32x16 pa, pb;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const bool last = 8 * (i >> 2) + (i & 3) <= x;
            pa[i] = last ? 0.0f : t[i];
            pb[i] = last ? t[i] : 0.0f;
        }
        auto pv = [&](int h, const f32x16 &p, auto first_tag) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const bf16x8 pf = cfrag(p, u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk)
                    o[dblk] = mfma_bf16(ofrag_tr(vsm, lo, h, u, dblk), pf, (decltype(first_tag)::value && u == 0) ? zero16 : o[dblk]);
            }
        };
        pv(0, pa, std::true_type{});
#pragma unroll
        for (int h = 1; h < NH - 1; ++h) {
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const float e0 = fast_exp2(fmaf(s[h][i], c, nm)), e1 = fast_exp2(fmaf(s[h][i + 1], c, nm));
                s[h][i] = e0; s[h][i + 1] = e1;
                rs0 += e0; rs1 += e1;
            }
            pv(h, s[h], std::false_type{});
        }
        pv(NH - 1, pb, std::false_type{});
        l = rs0 + rs1;
    } else {
        // general test: key k0 + 32 h + rc + 4 half is visible to row r0 + l32 iff it is not in front of key 0, not
        // after the row and less than W behind it: lo_l <= 32 h + rc <= x + W
        const int lo_l = max(x + 1, -k0 - 4 * half);
        const unsigned width = (unsigned)(x + W - lo_l);
        float mx0 = -INFINITY, mx1 = -INFINITY;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const int rc = 32 * h + 8 * (i >> 2) + (i & 3);
                s[h][i] = (unsigned)(rc - lo_l) <= width ? s[h][i] : -INFINITY;
                s[h][i + 1] = (unsigned)(rc + 1 - lo_l) <= width ? s[h][i + 1] : -INFINITY;
                mx0 = fast_max(mx0, s[h][i]);
                mx1 = fast_max(mx1, s[h][i + 1]);
            }
        m = fast_max(sink2, xhalf_max(fast_max(mx0, mx1)) * c);
        m = no_keys ? sink2 : m;
        const float nm = no_keys ? -INFINITY : -m;

        float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
        for (int h = 0; h < NH; ++h) {
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const float e0 = fast_exp2(fmaf(s[h][i], c, nm)), e1 = fast_exp2(fmaf(s[h][i + 1], c, nm));
                s[h][i] = e0; s[h][i + 1] = e1;
                rs0 += e0; rs1 += e1;
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const bf16x8 pf = cfrag(s[h], u);
#pragma unroll
                for (int dblk = 0; dblk < 2; ++dblk)
                    o[dblk] = mfma_bf16(ofrag_tr(vsm, lo, h, u, dblk), pf, (h == 0 && u == 0) ? zero16 : o[dblk]);
            }
        }
        l = rs0 + rs1;
    }

    // epilogue: z = l + exp(sink - m); O = acc / z; M = m + log z   (ref :93-98).  The output rows go through the K
    // buffer once nobody reads it any more.
    __syncthreads();
    const float z = xhalf_sum(l) + fast_exp2(sink2 - m);
    const float inv = 1.0f / z;
    bf16 *stage = reinterpret_cast<bf16 *>(smem) + w * 32 * kLS;
#pragma unroll
    for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            bf16x4 pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = (bf16)(o[dblk][4 * a4 + e] * inv);
            *reinterpret_cast<bf16x4 *>(stage + l32 * kLS + 32 * dblk + 8 * a4 + 4 * half) = pk;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    {
        // whole 128-byte rows, eight per store instruction
        char *oblk = reinterpret_cast<char *>(a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)r0 * a.os.s);
        const int cc = lane & 7, rr = lane >> 3;
        const uint32_t ooff = (uint32_t)(rr * (int)a.os.s + cc * 8) * 2u;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
            *reinterpret_cast<u32x4 *>(oblk + (int64_t)(8 * pass) * a.os.s * 2 + ooff) =
                *reinterpret_cast<const u32x4 *>(stage + (rr + 8 * pass) * kLS + cc * 8);
    }
    if (half == 0) a.lse[((int64_t)b * a.H + head) * a.Sq + r0 + l32] = (m + fast_log2(z)) * kLn2;
}

}  // namespace gptoss
