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
// Work split.  A workgroup is four query heads of one KV head (a wavefront each) on 64 query rows r0 .. r0 + 63, done as
// two blocks of 32 one after the other.  The keys r0 - W .. r0 + 63 (W + 64 rows of K and of V) are staged in LDS once
// for the four heads and both blocks, in one go; the second block's Q rows are requested while the first block's
// output is packed up, and that output is on its way to memory while the second block is computed.  (Problems too
// small to fill the chip that way are launched with one block per workgroup.)
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
    static constexpr int kRows = 32 * (NH + 1);    // rows of K (and of V) staged per workgroup: two query blocks' worth
    static constexpr int kTileBytes = kRows * kRowBytes;
    static constexpr int kStageBytes = 4 * 32 * kLS * 2;             // the four wavefronts' last output rows pass through the K buffer
    static constexpr int kKBytes = kTileBytes > kStageBytes ? kTileBytes : kStageBytes;
    static constexpr int kSmallStageBytes = 16 * kRowBytes;          // per wavefront: 16 output rows of the first query block
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
    // The stores recompute the lane index and what hangs on it, so that none of it has to live through the GEMMs in a
    // register file that is full there.
    auto fresh_lane = []() __attribute__((always_inline)) { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); };

    // workgroup (x, y, z) = (kv head, batch row and group of four query heads, pair of 32-row query blocks); workgroups
    // are dealt to the XCDs in x-fastest order, so that with G == 8 each XCD keeps one KV head's K / V in its own L2
    const int n_hc = a.r >> 2;
    const int g = blockIdx.x;
    const int b = blockIdx.y / n_hc, hc = blockIdx.y - b * n_hc;
    // the host launches one workgroup per pair of query blocks, or (small problems, which would leave compute units
    // idle) one per block: the grid says which
    const bool pairs = 32 * (int)gridDim.z < a.Sq;
    const int r0 = (pairs ? 64 : 32) * blockIdx.z; // first query row of the workgroup
    const int head = g * a.r + 4 * hc + w;
    const int k0 = r0 - W;                         // first staged key; negative for the first blocks of a row
    const bool two = pairs && r0 + 32 < a.Sq;      // (a row may end with a single block)
    // right-padded batch rows: query rows at or beyond the row's length have no keys (O = 0, lse = the sink logit); the
    // rows that exist never see a key beyond it
    const int len = a.seqlens ? min(max(a.seqlens[b], 0), a.Sq) : a.Sq;
    const float sink2 = (a.sinks ? a.sinks[head] : 0.0f) * kLog2e;

    char *const oblk0 = reinterpret_cast<char *>(a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)r0 * a.os.s);
    float *const lse0 = a.lse + ((int64_t)b * a.H + head) * a.Sq + r0;
    // lane's 16 bytes of an 8-row group of output rows: row lane / 8, piece lane % 8
    auto out_offset = [&](int ln) __attribute__((always_inline)) { return (uint32_t)((ln >> 3) * (int)a.os.s + (ln & 7) * 8) * 2u; };
    // a query block of nothing but padding: zeros, and the lse the arithmetic below gives a row without keys
    auto padding_block = [&](int X) __attribute__((always_inline)) {
        const int ln = fresh_lane();
        const uint32_t ooff = out_offset(ln);
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
            *reinterpret_cast<u32x4 *>(oblk0 + (int64_t)(32 * X + 8 * pass) * a.os.s * 2 + ooff) = u32x4{0u, 0u, 0u, 0u};
        if (ln < 32) lse0[32 * X + ln] = (sink2 + fast_log2(1.0f)) * kLn2;
    };
    if (r0 >= len) {
        padding_block(0);
        if (two) padding_block(1);
        return;
    }
    const bool live1 = two && r0 + 32 < len;       // the second block has rows that exist

    bf16x8 qf[4];                                  // Q^T fragments (B operand) of the block at hand
    const char *const qblk0 = reinterpret_cast<const char *>(a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)r0 * a.qs.s);
    auto load_q = [&](int X) __attribute__((always_inline)) {
        const int ln = fresh_lane();
        const uint32_t qoff = (uint32_t)((ln & 31) * (int)a.qs.s + 8 * (ln >> 5)) * 2u;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
            qf[ks] = as_bf16x8(*reinterpret_cast<const u32x4 *>(qblk0 + (int64_t)(32 * X) * a.qs.s * 2 + qoff + 32 * ks));
    };
    load_q(0);
    const uint32_t ksm = lds_addr(smem), vsm = ksm + C::kKBytes;
    {
        // copy j of wavefront w fills rows 8 (w + 4 j) .. + 7 of the staged range (the second block's own 32 keys, j = NH,
        // only where that block exists); rows in front of key 0 re-read key 0 (their logits are masked, they only have
        // to be finite)
        const int rloc = 8 * w + (lane >> 3);
        const int ch = (lane & 7) ^ swz(rloc);     // swz() of the row: 32 j does not reach the bits it looks at
        const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h, *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;
        char *kdst = smem + w * 8 * kRowBytes, *vdst = smem + C::kKBytes + w * 8 * kRowBytes;
        // addresses are (scalar pointer) + (32-bit lane offset): the row of copy j is a scalar step away from copy 0's,
        // except where rows are held at key 0
        auto copy_all = [&](const bf16 *base, int stride, char *dst) __attribute__((always_inline)) {
            if (k0 >= 0) {
                const uint32_t voff = (uint32_t)(rloc * stride + ch * 8) * 2u;
#pragma unroll
                for (int j = 0; j <= NH; ++j)
                    if (j < NH || live1)
                        __builtin_amdgcn_global_load_lds((glb_void_t *)(reinterpret_cast<const char *>(base + (int64_t)(k0 + 32 * j) * stride) + voff),
                                                         (lds_void_t *)(dst + j * 32 * kRowBytes), 16, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j <= NH; ++j)
                    if (j < NH || live1) {
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
    const TileLaneOffsets lo = make_tile_offsets(lane);
    const int x = l32 - 4 * half;                  // register i of a block holds key rc(i) + 4 half: "key <= row" is rc(i) <= x
    const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};

    wait_vmcnt<0>();                               // this wavefront's copies of K and V (and its Q rows) have landed ...
    __syncthreads();                               // ... and everybody else's

    // One query block, X = 0 or 1: rows r0 + 32 X .., keys in the staged blocks X .. X + NH - 1.  Leaves the unscaled
    // output in o, the row's reference m and this lane's share l of the row sum.
    f32x16 o[2];
    float m, l;
    auto block = [&](auto x_tag) __attribute__((always_inline)) {
        constexpr int X = decltype(x_tag)::value;
        const bool edge = k0 + 32 * X < 0;
        const bool no_keys = r0 + 32 * X + l32 >= len;          // this lane's row is padding
        // S^T = K Q^T for all NH blocks: lane = query row l32, register i of block h = key 32 h + rc(i) + 4 half
        f32x16 s[NH];
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            s[h] = mfma_bf16(ofrag_nat(ksm, lo, X + h, 0), qf[0], zero16);
#pragma unroll
            for (int ks = 1; ks < 4; ++ks) s[h] = mfma_bf16(ofrag_nat(ksm, lo, X + h, ks), qf[ks], s[h]);
        }
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
                        o[dblk] = mfma_bf16(ofrag_tr(vsm, lo, X + h, u, dblk), pf, (decltype(first_tag)::value && u == 0) ? zero16 : o[dblk]);
                }
            };
            pv(0, pa, std::true_type{});
            pv(NH - 1, pb, std::false_type{});
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
            l = rs0 + rs1;
        } else {
            // general test: key k0 + 32 (X + h) + rc + 4 half is visible to row r0 + 32 X + l32 iff it is not in front of
            // key 0, not after the row and less than W behind it: lo_l <= 32 h + rc <= x + W
            const int lo_l = max(x + 1, -(k0 + 32 * X) - 4 * half);
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
                        o[dblk] = mfma_bf16(ofrag_tr(vsm, lo, X + h, u, dblk), pf, (h == 0 && u == 0) ? zero16 : o[dblk]);
                }
            }
            l = rs0 + rs1;
        }
    };

    // Results: z = l + exp(sink - m); O = acc / z; M = m + log z   (ref :93-98).  The output rows leave as whole
    // 128-byte rows, eight per store instruction, which takes a trip through LDS.
    // The workgroup's last block (everybody is past the barrier, the K buffer is free): 32 padded rows per wavefront.
    auto store_last = [&](int X) __attribute__((always_inline)) {
        const float z = xhalf_sum(l) + fast_exp2(sink2 - m);
        const float inv = 1.0f / z;
        const int ln = fresh_lane(), row = ln & 31, hf = ln >> 5, cc = ln & 7, rr = ln >> 3;
        const uint32_t ooff = out_offset(ln);
        bf16 *stage = reinterpret_cast<bf16 *>(smem) + w * 32 * kLS;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                bf16x4 pk;
#pragma unroll
                for (int e = 0; e < 4; ++e) pk[e] = (bf16)(o[dblk][4 * a4 + e] * inv);
                *reinterpret_cast<bf16x4 *>(stage + row * kLS + 32 * dblk + 8 * a4 + 4 * hf) = pk;
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int pass = 0; pass < 4; ++pass)
            *reinterpret_cast<u32x4 *>(oblk0 + (int64_t)(32 * X + 8 * pass) * a.os.s * 2 + ooff) =
                *reinterpret_cast<const u32x4 *>(stage + (rr + 8 * pass) * kLS + cc * 8);
        if (hf == 0) lse0[32 * X + row] = (m + fast_log2(z)) * kLn2;
    };
    // The first block while the second still needs the staged rows: only the first 32 rows of K and of V are free (the
    // second block starts one 32-key block later), 2 KB per wavefront, so the rows go in two halves of 16, unpadded,
    // with the 16-byte pieces of a row rotated by the row number against bank conflicts.
    auto store_first = [&]() __attribute__((always_inline)) {
        const float z = xhalf_sum(l) + fast_exp2(sink2 - m);
        const float inv = 1.0f / z;
        const int ln = fresh_lane(), row32 = ln & 31, hf = ln >> 5, cc = ln & 7, rr = ln >> 3;
        const uint32_t ooff = out_offset(ln);
        char *stage = smem + (w >> 1) * C::kKBytes + (w & 1) * C::kSmallStageBytes;   // wavefronts 0, 1 in K's rows, 2, 3 in V's
        uint32_t pk[8][2];
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                union { bf16x4 v; uint32_t u[2]; } cv;
#pragma unroll
                for (int e = 0; e < 4; ++e) cv.v[e] = (bf16)(o[dblk][4 * a4 + e] * inv);
                pk[4 * dblk + a4][0] = cv.u[0];
                pk[4 * dblk + a4][1] = cv.u[1];
            }
        const int row16 = row32 & 15;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if ((row32 >> 4) == p) {
#pragma unroll
                for (int piece = 0; piece < 8; ++piece) {
                    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
                    *reinterpret_cast<u32x2 *>(stage + row16 * kRowBytes + ((piece ^ (row16 & 7)) * 16) + 8 * hf) = u32x2{pk[piece][0], pk[piece][1]};
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int row = rr + 8 * q;
                *reinterpret_cast<u32x4 *>(oblk0 + (int64_t)(16 * p + 8 * q) * a.os.s * 2 + ooff) =
                    *reinterpret_cast<const u32x4 *>(stage + row * kRowBytes + ((cc ^ (row & 7)) * 16));
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        if (hf == 0) lse0[row32] = (m + fast_log2(z)) * kLn2;
    };

    block(std::integral_constant<int, 0>{});
    __syncthreads();                               // nobody reads the first 32 staged rows any more; without a second block, any of them
    if (!live1) {
        store_last(0);
        if (two) padding_block(1);
        return;
    }
    load_q(1);                                     // the second block's Q rows travel while the first block's results are packed up
    store_first();
    block(std::integral_constant<int, 1>{});
    __syncthreads();
    store_last(1);
}

}  // namespace gptoss
