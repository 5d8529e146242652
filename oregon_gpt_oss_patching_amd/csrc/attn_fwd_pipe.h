// Forward kernel for the plain full-causal case (bf16, no window, no packed rows, no query offset, right-padded
// batch rows allowed, Sq == Skv a multiple of 64, query heads per KV head a multiple of 4): the formulas of
// attn_fwd_kernel<4, 2> (attn_fwd.h; the reference's `_attn_fwd`, attention_kernel.py:11-100) with the
// interior key tiles software-pipelined by hand.  Against that kernel only the order of the row sums of a
// row's first tile differs: lse agrees to a few units of its last place, O to one bf16 rounding.
//
// Why.  Two wavefronts share a SIMD.  attn_fwd_kernel's wavefront issues its MFMAs in clumps of eight with a
// softmax step (about 120 vector instructions, no MFMA) between them; while one wavefront sits in such a
// vector stretch the matrix pipe has only the other one to feed it, and when both do, it idles.  An
// instruction stream in which every MFMA is followed by its share of the vector work keeps both pipes
// supplied whatever the phase of the neighbour: measured with synthetic streams of the forward's
// instruction mix at two wavefronts per SIMD, 53.6 cycles per MFMA against 58.8 for the clumped order.
//
// How.  A tile is four units u = (32-key block kb, 32-row block qb).  Slot u issues, as eight micro-slots
// of {one MFMA, two elements of softmax, at most two LDS reads} closed by sched_barrier(0):
//   * the four S MFMAs of unit u + 1 (the next tile's first unit in the tile's last slot),
//   * the four O += P V MFMAs of unit u - 1,
//   * exp2 / row sum / bf16 packing of unit u's sixteen logits per lane.
// K fragments (natural) and V fragments (transposed) each feed both row blocks and are reloaded in place
// right after their last use, one slot before their first.  The next tile must have landed before the
// third slot of a tile (which loads its first K fragments), so the iteration's barrier sits there; with four
// LDS stages the copy requested at that barrier is two tiles ahead, as in attn_fwd_kernel.
// The softmax reference of a row (see fwd_tile_lean) is the sink logit or the largest logit of the row's first
// tile, taken by a pass over that tile that forms the logits and nothing else; the tile then goes through the
// loop like the others.  The diagonal tile (masked) goes through attn_fwd.h's fwd_tile_lean; rows of a single
// key tile, and the rare second pass of a workgroup whose frozen reference turned out too low, go through one
// loop of exact steps (fwd_tile).
#pragma once
#include <type_traits>

#include "attn_fwd.h"

namespace gptoss {

struct FwdPipe {
    static constexpr int NS = 4;                                  // LDS stages
    static constexpr int kStageBytes = 2 * kStageTileBytes;       // K tile, V tile
};

// PADDED: right-padded batch rows (seqlens): a row of the batch is a shorter row.  Workgroups past its end write
// O = 0 and lse = sink and do nothing else; in the workgroup that holds its end the rows past it run along
// unmasked through the interior tiles (their logits are garbage but finite or at worst NaN, and stay in their own
// lanes) and are set to that same result before the epilogue; keys past the end exist only in the diagonal
// tile, whose tile function masks them.
template <bool PADDED>
__global__ __launch_bounds__(256, 2) void attn_fwd_pipe_kernel(const KArgs a) {
    constexpr int NS = FwdPipe::NS;
    constexpr int SB = FwdPipe::kStageBytes;
    __shared__ __attribute__((aligned(16))) char smem[NS][2][kStageTileBytes];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: the head and everything derived from it stay in scalar registers
    const int l32 = lane & 31, half = lane >> 5;
    // What follows the pipelined loop (the diagonal tile, the rare second pass, the epilogue) recomputes the lane
    // index and what hangs on it, so that none of it has to live through the loop in a register file that is full there.
    auto fresh_lane = []() __attribute__((always_inline)) { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); };

    // workgroup -> (kv head, chunk of 4 heads, batch, query tile), as attn_fwd_kernel; longest key loops first
    const int n_hc = a.r / 4;
    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int hc = bid % n_hc; bid /= n_hc;
    const int b = bid % a.B; bid /= a.B;
    const int qt = a.Sq / kTile - 1 - bid;
    const int head = g * a.r + hc * 4 + w;
    const int qw0 = qt * kTile;                    // the four wavefronts hold the same 64 rows of four heads
    const int n_it = qt + 1;                       // key tiles 0 .. qt, the last one on the diagonal
    const int len = PADDED ? max(0, min(a.Sq, a.seqlens[b])) : a.Sq;      // rows and keys from len on do not exist
    const bool wg_dead = PADDED && qw0 >= len;

    const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const bf16 *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;

    bf16x8 qf[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const int row = qw0 + 32 * qb + l32;
        const bf16 *qrow = a.q + (int64_t)b * a.qs.b + (int64_t)head * a.qs.h + (int64_t)row * a.qs.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qf[qb][ks] = as_bf16x8(*reinterpret_cast<const u32x4 *>(qrow + 16 * ks + 8 * half));
    }

    const float c = a.scale_log2;
    const float sink2 = (a.sinks ? a.sinks[head] : 0.0f) * kLog2e;
    float m[2], l[2];
    f32x16 o[2][2];

    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(&smem[0][0][0]);
    const AsyncLaneOffsets klane = make_async_offsets(a.ks.s, lane, w), vlane = make_async_offsets(a.vs.s, lane, w);
    const uint32_t copy_base = smem_base + w * (16 * kRowBytes);   // this wavefront copies rows 16 w .. 16 w + 15
    // Requests are branch-free (a branch inside the fenced loop body lets the compiler sink vector work of
    // earlier micro-slots past it): every arrive() is followed by exactly one request, and once the row's
    // tiles are exhausted a request copies the last tile again, into the stage that is free by then, so that
    // "at most one request outstanding" keeps meaning "the tile before it has landed".
    const bf16 *ktile = kbase, *vtile = vbase;
    int iss_stage = 0, iss_left = n_it;
    auto issue = [&]() __attribute__((always_inline)) {       // the next tile in order, into the next stage in rotation
        // (through the inline-assembly copy: the compiler's own bookkeeping would make every LDS read that
        // follows a copy wait for all outstanding copies, i.e. for the tile just requested)
        const uint32_t dst = copy_base + iss_stage * SB;
        lds_dma16_plus<0>(dst, ktile, klane.off[0]);
        lds_dma16_plus<8 * kRowBytes>(dst, ktile, klane.off[1]);
        lds_dma16_plus<kStageTileBytes>(dst, vtile, vlane.off[0]);
        lds_dma16_plus<kStageTileBytes + 8 * kRowBytes>(dst, vtile, vlane.off[1]);
        const bool more = iss_left > 1;
        ktile += more ? kTile * a.ks.s : 0;
        vtile += more ? kTile * a.vs.s : 0;
        iss_left -= 1;
        iss_stage = (iss_stage + 1) & (NS - 1);
    };
    constexpr int kLoadsPerIt = 4;
    auto reset = [&]() __attribute__((always_inline)) {
        ktile = kbase;
        vtile = vbase;
        iss_stage = 0;
        iss_left = n_it;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            m[qb] = sink2;
            l[qb] = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) { o[qb][0][i] = 0.0f; o[qb][1][i] = 0.0f; }
        }
        issue();
        issue();
    };
    // tile k has landed in every wavefront (the k-th call); the stage of tile k - 2 is free and takes tile k + 2
    auto arrive = [&]() __attribute__((always_inline)) {
        wait_vmcnt<kLoadsPerIt>();
        __syncthreads();
        issue();
    };
    // Rows of a single key tile (the diagonal one) have no interior tile: they go straight to the exact pass below.
    const bool pipelined = !wg_dead && n_it >= 2;
    if (!pipelined) {
        // (also the state a workgroup without rows ends with: nothing requested, nothing attended)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            m[qb] = sink2;
            l[qb] = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) { o[qb][0][i] = 0.0f; o[qb][1][i] = 0.0f; }
        }
    } else {
        reset();
        arrive();
        // The softmax reference of a row: the sink logit or the largest logit of the row's first tile
        // (ref :53, :79-81 after one tile), from a pass over that tile that forms the logits and nothing else
        // (16 MFMAs per row block, against 32 for each of its tiles).  The tile then goes through the pipelined
        // loop like every other interior tile.
        f32x16 s[2][2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const bf16x8 akf = ofrag_nat(smem_base, lo, kb, ks);
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    f32x16 z;
#pragma unroll
                    for (int i = 0; i < 16; ++i) z[i] = 0.0f;
                    s[kb][qb] = mfma_bf16(akf, qf[qb][ks], ks == 0 ? z : s[kb][qb]);
                }
            }
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            float mx0 = s[0][qb][0], mx1 = s[1][qb][0];
#pragma unroll
            for (int i = 1; i < 16; ++i) { mx0 = fast_max(mx0, s[0][qb][i]); mx1 = fast_max(mx1, s[1][qb][i]); }
            m[qb] = fast_max(m[qb], xhalf_max(fast_max(mx0, mx1)) * c);
        }
    }
    float nm[2] = {-m[0], -m[1]};

    if (pipelined) {
#define GPTOSS_FP_FENCE() __builtin_amdgcn_sched_barrier(0)
        // (an MFMA's result is not needed before the next slot, and instruction selection would place it there,
        // across the fences, which only bind the scheduler that runs afterwards: an empty volatile statement
        // that takes the result as an operand keeps the MFMA inside its micro-slot)
#define GPTOSS_FP_PIN(x) asm volatile("" : "+v"(x))
        // ---- pipeline state ----
        f32x16 sa, sb;                      // logits of the unit in the softmax / of the unit being multiplied
        bf16x8 pa[2], pb[2];                // [u16] P of the unit in the softmax / of the unit before it
        bf16x8 ak[4];                       // [ks] K fragments of the key block whose S is being formed
        bf16x8 av[2][2];                    // [u16][dblk] V fragments of the key block being multiplied into O
        uint32_t kadr[4], vadr[2][2];       // per-lane LDS addresses: K of the stage the next K fragments come from, V of this tile's
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) kadr[ks] = smem_base + lo.nat[ks];                      // tile 0 is in stage 0
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) vadr[dblk][t2] = smem_base + kStageTileBytes + lo.tr[dblk][t2];
        // fill: S of unit 0 of tile 0; the first slot's O MFMAs multiply zeros (O is zero there anyway)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) ak[ks] = as_bf16x8(lds_load128(kadr[ks], 0));
#pragma unroll
        for (int u16 = 0; u16 < 2; ++u16) {
#pragma unroll
            for (int e = 0; e < 8; ++e) { pb[u16][e] = (bf16)0.0f; av[u16][0][e] = (bf16)0.0f; av[u16][1][e] = (bf16)0.0f; }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            f32x16 z;
#pragma unroll
            for (int i = 0; i < 16; ++i) z[i] = 0.0f;
            sa = mfma_bf16(ak[ks], qf[0][ks], ks == 0 ? z : sa);
        }
        GPTOSS_FP_FENCE();

        // slot U of a tile: softmax of unit U (logits s_cur -> P pf_cur), S of unit U + 1 (-> s_next), O += P V of unit U - 1 (pf_prev)
        auto slot = [&](auto u_, f32x16 &s_cur, f32x16 &s_next, bf16x8 (&pf_prev)[2], bf16x8 (&pf_cur)[2]) __attribute__((always_inline)) {
            constexpr int U = decltype(u_)::value;
            constexpr int qb = U & 1, qo = qb ^ 1;            // the units before and after U are of the other row block
            constexpr bool RELOAD = (U & 1) == 0;             // they are the last users of the fragments in registers
            float rs0 = 0.0f, rs1 = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int i = j >> 1;
                if ((j & 1) == 0) {
                    f32x16 z;
#pragma unroll
                    for (int e = 0; e < 16; ++e) z[e] = 0.0f;
                    s_next = mfma_bf16(ak[i], qf[qo][i], i == 0 ? z : s_next);
                    GPTOSS_FP_PIN(s_next);
                    // U == 0: key block 1 of this tile; U == 2: key block 0 of the next one (kadr is there already)
                    if (RELOAD) ak[i] = as_bf16x8(lds_load128(kadr[i], U == 0 ? 32 * kRowBytes : 0));
                } else {
                    const int u16 = i >> 1, dblk = i & 1;
                    o[qo][dblk] = mfma_bf16(av[u16][dblk], pf_prev[u16], o[qo][dblk]);
                    GPTOSS_FP_PIN(o[qo][dblk]);
                    if (RELOAD) {                             // the V fragments of unit U's own key block
                        const int imm = (32 * (U >> 1) + 16 * u16) * kRowBytes;
                        union { struct { s16x4 a, b; } s; bf16x8 v; } x;
                        x.s.a = lds_load_tr64(vadr[dblk][0], imm);
                        x.s.b = lds_load_tr64(vadr[dblk][1], imm);
                        av[u16][dblk] = x.v;
                    }
                }
                const float e0 = fast_exp2(fmaf(s_cur[2 * j], c, nm[qb])), e1 = fast_exp2(fmaf(s_cur[2 * j + 1], c, nm[qb]));
                rs0 += e0;
                rs1 += e1;
                pf_cur[j >> 2][(2 * j) & 7] = (bf16)e0;
                pf_cur[j >> 2][((2 * j) & 7) + 1] = (bf16)e1;
                GPTOSS_FP_FENCE();
            }
            l[qb] += rs0 + rs1;
        };
        using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;

        // (whatever loads the compiler itself has in flight here, reloads of spilled registers included, are
        // known to have arrived after this wait, so it puts no vmcnt wait of its own into the loop, where it
        // would also wait for the copies in flight)
        // (the Q fragments, which the first tile's exact step pushes out to scratch, are asked for here so that
        // their reloads come before the wait rather than after it)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) asm volatile("" ::"v"(qf[qb][ks]));
        wait_vmcnt<0>();
        for (int t = 0; t <= n_it - 2; ++t) {
            GPTOSS_FP_FENCE();
            slot(I0{}, sa, sb, pb, pa);
            slot(I1{}, sb, sa, pa, pb);
            // the next tile has landed; its first K fragments are loaded in the slot that follows, its V fragments
            // from the next pass of this loop on
            arrive();
            const uint32_t step = ((t + 1) & (NS - 1)) ? (uint32_t)SB : (uint32_t)(SB - NS * SB);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) kadr[ks] += step;
            GPTOSS_FP_FENCE();
            slot(I2{}, sa, sb, pb, pa);
            slot(I3{}, sb, sa, pa, pb);
#pragma unroll
            for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
                for (int t2 = 0; t2 < 2; ++t2) vadr[dblk][t2] += step;
        }
        // drain: O += P V of the last pipelined tile's last unit (sa holds S of the diagonal tile's first unit,
        // which the masked tile function below forms again with the mask)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int u16 = i >> 1, dblk = i & 1;
            o[1][dblk] = mfma_bf16(av[u16][dblk], pb[u16], o[1][dblk]);
        }
        GPTOSS_FP_FENCE();
#undef GPTOSS_FP_FENCE
#undef GPTOSS_FP_PIN
    }
    const int lane_b = fresh_lane(), l32_b = lane_b & 31, half_b = lane_b >> 5;
    const TileLaneOffsets lo_b = make_tile_offsets(lane_b);
    int pq_b[2];
    unsigned wl_b[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) { pq_b[qb] = qw0 + 32 * qb + l32_b < len ? qw0 + 32 * qb + l32_b : -0x40000000; wl_b[qb] = 0x3fffffffu; }   // (hugely negative: nothing is visible to a row that does not exist)
    auto masked_args_b = [&](int n0, int (&dbase)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) dbase[qb] = pq_b[qb] - n0;
    };
    if (pipelined) {
        const int n0 = qt * kTile;
        const uint32_t ksm = smem_base + (qt & (NS - 1)) * SB;
        int dbase[2];
        masked_args_b(n0, dbase);
        fwd_tile_lean<true, 2>(ksm, ksm + kStageTileBytes, lo_b, qf, o, nm, l, c, lane_b, dbase, wl_b, 0x3fffffffu, len - n0, 0);
    }

    // A sum beyond 2^96 (or not finite): some logit stood 95 or more above its row's frozen reference; the
    // workgroup repeats its key loop with the exact online-softmax step on every tile (see attn_fwd_kernel).
    // rows that do not exist: nothing attended, whatever the interior tiles made of them
    auto clear_dead_rows = [&]() __attribute__((always_inline)) {
        if constexpr (PADDED) {
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
                const bool dead_row = pq_b[qb] < 0;
                m[qb] = dead_row ? sink2 : m[qb];
                l[qb] = dead_row ? 0.0f : l[qb];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    o[qb][0][i] = dead_row ? 0.0f : o[qb][0][i];
                    o[qb][1][i] = dead_row ? 0.0f : o[qb][1][i];
                }
            }
        }
    };
    clear_dead_rows();
    // A sum beyond 2^96 (or not finite): some logit stood 95 or more above its row's frozen reference; the
    // workgroup repeats its key loop with the exact online-softmax step on every tile (see attn_fwd_kernel; the
    // masked form of the step for every tile: this pass is rare and the kernel stays small).  Rows of a single
    // tile take this pass as their only one.
    bool unsafe = false;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) unsafe = unsafe || !(l[qb] < 0x1p96f);
    const bool second_pass = pipelined && __syncthreads_or(unsafe);
    if (second_pass || (!pipelined && !wg_dead)) {
        if (second_pass) {
            wait_vmcnt<0>();      // the repeated copies of the last requests
            __syncthreads();
        }
        reset();
        for (int it = 0; it < n_it; ++it) {
            arrive();
            const uint32_t ksm = smem_base + (it & (NS - 1)) * SB;
            int dbase[2];
            masked_args_b(it * kTile, dbase);
            fwd_tile<true, 2>(ksm, ksm + kStageTileBytes, lo_b, qf, o, m, l, c, lane_b, dbase, wl_b, 0x3fffffffu, len - it * kTile, qw0 - it * kTile);
        }
        clear_dead_rows();
    }

    // epilogue: z = l + exp(sink - m); O = acc / z; M = m + log z   (ref :93-98)
    wait_vmcnt<0>();              // the repeated copies of the last requests
    __syncthreads();
    bf16 *stage = reinterpret_cast<bf16 *>(&smem[0][0][0]) + w * 32 * kLS;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const float l_tot = l[qb] + __shfl_xor(l[qb], 32);
        const float z = l_tot + fast_exp2(sink2 - m[qb]);
        const float inv = 1.0f / z;
        const int r0 = qw0 + 32 * qb;
        bf16 *orow0 = a.o + (int64_t)b * a.os.b + (int64_t)head * a.os.h + (int64_t)r0 * a.os.s;
        store_rows32(stage, o[qb], inv, orow0, a.os.s, a.Sq - r0, lane_b);
        __builtin_amdgcn_wave_barrier();
        if (half_b == 0) a.lse[((int64_t)b * a.H + head) * a.Sq + r0 + l32_b] = (m[qb] + fast_log2(z)) * kLn2;
    }
}

}  // namespace gptoss
