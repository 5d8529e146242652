// Single-pass backward for sliding-window layers (window <= 128): dQ, dK, dV and the dSinks
// terms from ONE read of Q, dO, O, K, V, five GEMMs per (query tile, key tile) pair.  Stands in for
// the reference's `_attn_bwd_precompute_D` + `_attn_bwd` (attention_kernel.py:102-217) on such
// layers; results are bit-reproducible (no atomics, fixed summation orders).
//
// With a window of at most 128 a 64-row query tile t sees the three 64-key tiles t-2, t-1, t,
// and a key tile is seen by the query tiles t, t+1, t+2.  A workgroup owns a chunk of
// consecutive query tiles [t0, t1) of one KV head (all r query heads of the group) and walks
// (query tile, head), heads inner.  Eight wavefronts:
//   * six "owners", in three pairs; pair p holds, as MFMA B operands in registers, the K and V
//     rows of the one live key tile kt with kt % 3 == p (32 keys per wavefront) and that tile's
//     dK / dV accumulators.  Per iteration an owner does what the dK/dV kernel does for its keys
//     (S = Q K^T, dP = dO V^T, P, dS, dV^T += dO^T P, dK^T += Q^T dS; see dkdv_tile) and leaves the
//     bf16 dS block in LDS, key-major.  When the walk moves on to query tile t, key tile t-3 is
//     complete: its pair writes dK / dV out and takes over key tile t.
//   * two "helpers".  Helper hh owns rows 32*hh .. 32*hh+31 of every query tile: one iteration
//     AHEAD of the owners it forms the row statistics lse*log2(e) and -rowsum(dO*O) of its rows
//     (from O and dO rows it reads itself) and leaves them in LDS; one iteration BEHIND them it
//     turns the dS tile into dQ^T = K^T dS^T over all 192 live keys (K fragments of the three live
//     key tiles resident in its registers) and writes the finished dQ rows.  It also sums the
//     dSinks terms exp(sink - lse) * (-delta) of its rows.
// All 192 keys a query tile can see are in the workgroup at the same time, so dQ is complete
// when the helper stores it.  A key tile collects from three query tiles, so the last two key
// tiles of a chunk (and the two before it, which the chunk walks for the sake of its first rows'
// dQ) are completed by two neighbouring workgroups.  Two ways of closing that seam:
//   * boundary_partial set (gptoss_attn_bwd): each of the two workgroups leaves its fp32 share of
//     dK / dV of those tiles in the scratch, and attn_bwd_window_finish_kernel adds the two shares
//     in a fixed order, scales and rounds: 64 KB of partial sums per seam and tile pair, and a
//     walk of exactly the chunk's own query tiles;
//   * boundary_partial NULL (gptoss_attn_bwd_static, which has no room for the partial sums): the
//     walk goes two query tiles past the chunk, for the sake of its last two key tiles only, and
//     drops the dK / dV of the two key tiles before the chunk (the neighbour produces them the
//     same way): recomputation instead of an exchange, 25 % more iterations at 8 tiles per chunk.
// Both are free of atomics and bit-reproducible.
//
// One barrier per iteration hands over the staged Q / dO tile (asynchronous global->LDS copies,
// three stages), the row statistics of the next tile and the dS tile of the previous one (double
// buffered).  K / V rows of the next key tile travel through an LDS transit buffer one query
// tile ahead of their use.
#pragma once
#include <type_traits>

#include "attn_bwd.h"
#include "attn_common.h"

namespace gptoss {

struct WinCfg {
    static constexpr int NOWN = 6, NHELP = 2, NWAVES = NOWN + NHELP, NS = 3;
    static constexpr int kMaxWindow = 128;
    static constexpr int kMaxGroup = 16;                                   // query heads per KV head
    static constexpr int kStageOff = 0;                                    // [NS][Q, dO][8 KB]
    static constexpr int kStatOff = kStageOff + NS * 2 * kStageTileBytes;  // [NS][lse2, -delta][64] floats
    static constexpr int kDsOff = kStatOff + NS * 2 * kTile * 4;           // [2][3 slabs of 64 keys][8 KB]
    static constexpr int kDsBytes = 3 * kStageTileBytes;
    static constexpr int kTransitOff = kDsOff + 2 * kDsBytes;              // [K, V][8 KB] of the next key tile
    static constexpr int kOutOff = kTransitOff + 2 * kStageTileBytes;      // [NWAVES][32 x kLS] bf16 output stages
    static constexpr int kSinkOff = kOutOff + NWAVES * 32 * kLS * 2;       // [NHELP][kMaxGroup][64 lanes] floats
    static constexpr int kLdsBytes = kSinkOff + NHELP * kMaxGroup * 64 * 4;
    static_assert(kDsOff % 128 == 0 && kTransitOff % 128 == 0, "swizzled tiles start on 128-byte boundaries");
    static_assert(kLdsBytes <= 160 * 1024, "one workgroup per CU");
    static_assert(kMaxGroup * NHELP * 64 * 4 == kLdsBytes - kSinkOff, "the dSinks slots in LDS bound the query heads per KV head");
};

// (query tile, head within the group) of a position of the walk
struct WinPos {
    int t, h;
    __device__ __forceinline__ void step(int r) { if (++h == r) { h = 0; ++t; } }
};

__global__ __launch_bounds__(WinCfg::NWAVES * 64, 1) void attn_bwd_window_kernel(const KArgs a) {
    using C = WinCfg;
    constexpr int NS = C::NS;
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    char *const smem = lds + C::kStageOff;
    float *const sstat = reinterpret_cast<float *>(lds + C::kStatOff);
    char *const dsbuf = lds + C::kDsOff;
    char *const transit = lds + C::kTransitOff;
    float *const ssink = reinterpret_cast<float *>(lds + C::kSinkOff);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps everything derived from it in scalar registers
    const int l32 = lane & 31, half = lane >> 5;
    const bool owner = w < C::NOWN;

    int bid = blockIdx.x;
    const int g = bid % a.G; bid /= a.G;
    const int b = bid % a.B; bid /= a.B;
    const int chunk = bid;
    const int n_chunks = gridDim.x / (a.G * a.B);
    const int nT = (a.Sq + kTile - 1) / kTile;
    const int t0 = chunk * a.chunk_tiles;                  // first query tile (and first own key tile)
    const int t1 = min(t0 + a.chunk_tiles, nT);            // end of the chunk
    const bool seam_sums = a.boundary_partial != nullptr;  // see the file comment
    const int t_end = seam_sums ? t1 : min(t1 + 2, nT);    // without them two more query tiles complete the chunk's dK / dV
    const int n_it = (t_end - t0) * a.r;

    const int kv_len = a.seqlens ? min(a.Skv, a.seqlens[b]) : a.Skv;
    const int q_len = a.seqlens ? a.seqlens[b] : 0x7fffffff;
    const int weff = a.window;

    const TileLaneOffsets lo = make_tile_offsets(lane);
    const uint32_t smem_base = lds_addr(smem), stat_base = lds_addr(sstat), ds_base = lds_addr(dsbuf);
    const uint32_t transit_base = lds_addr(transit);
    const bf16 *kbase = a.k + (int64_t)b * a.ks.b + (int64_t)g * a.ks.h;
    const bf16 *vbase = a.v + (int64_t)b * a.vs.b + (int64_t)g * a.vs.h;
    bf16 *const out_stage = reinterpret_cast<bf16 *>(lds + C::kOutOff) + w * 32 * kLS;

    // key tile that pair / slot p holds while the walk is at query tile t: the one of t-2, t-1, t
    // that is congruent to p modulo 3
    auto tile_of_slot = [](int p, int t) { return t - ((t - p) % 3 + 3) % 3; };

    // ---- prologue: the three key tiles live at the first query tile --------------------------
    // Their K rows go through LDS (slab p of the first dS buffer) so that the helpers can pick
    // them up as transposed fragments; rows outside the tensor repeat a valid row (finite values
    // that only ever meet dS = 0).
    for (int slot = w; slot < 24; slot += C::NWAVES) {
        const int p = slot >> 3, r8 = slot & 7;
        const int kt = tile_of_slot(p, t0);
        const int rr = 8 * r8 + (lane >> 3);
        const int cc = (lane & 7) ^ swz(rr);
        const int row = min(max(kt * kTile + rr, 0), a.Skv - 1);
        __builtin_amdgcn_global_load_lds((glb_void_t *)(kbase + (int64_t)row * a.ks.s + cc * 8),
                                         (lds_void_t *)(dsbuf + p * kStageTileBytes + r8 * 8 * kRowBytes), 16, 0, 0);
    }

    if (!owner) {
        // the two helpers are the only wavefronts of their kind; whenever one of them can issue it goes
        // before the owner it shares its SIMD with (measured: -4 % at S = 16384)
        __builtin_amdgcn_s_setprio(1);
        // =================================== helper wavefronts ===================================
        const int hh = w - C::NOWN;
        const int srow = 32 * hh + (lane >> 1), hr = lane & 1;     // statistics: two lanes per row, 32 columns each
        // dSinks terms are summed per lane (own LDS slot per head, no cross-lane traffic in the loop)
        float *const my_sink = ssink + (hh * C::kMaxGroup) * 64 + lane;
        for (int h = 0; h < a.r; ++h) my_sink[h * 64] = 0.0f;
        const float *sinks = a.sinks;

        // O and dO half rows + lse of this lane's row of walk position `pos`.  The row pointers
        // follow the walk (heads inner, then the next query tile); the last tile's rows past the
        // end of the tensor re-read the last valid row.
        u32x4 pre_o[4], pre_g[4];
        float pre_lse = 0.0f;
        const int64_t stat_row0 = min(t0 * kTile + srow, a.Sq - 1);
        const bf16 *orow = a.o + (int64_t)b * a.os.b + (int64_t)(g * a.r) * a.os.h + stat_row0 * a.os.s + 32 * hr;
        const bf16 *grow = a.d_o + (int64_t)b * a.dos.b + (int64_t)(g * a.r) * a.dos.h + stat_row0 * a.dos.s + 32 * hr;
        const float *lrow = a.lse + ((int64_t)b * a.H + (int64_t)g * a.r) * a.Sq + stat_row0;
        auto prefetch = [&](WinPos &pos) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                pre_o[j] = *reinterpret_cast<const u32x4 *>(orow + 8 * j);
                pre_g[j] = *reinterpret_cast<const u32x4 *>(grow + 8 * j);
            }
            pre_lse = *lrow;
            orow += a.os.h;
            grow += a.dos.h;
            lrow += a.Sq;
            if (++pos.h == a.r) {
                pos.h = 0;
                ++pos.t;
                // rows of the next tile (clamped at the end of the tensor)
                const int64_t adv = min(pos.t * kTile + srow, a.Sq - 1) - min((pos.t - 1) * kTile + srow, a.Sq - 1);
                orow += adv * a.os.s - (int64_t)a.r * a.os.h;
                grow += adv * a.dos.s - (int64_t)a.r * a.dos.h;
                lrow += adv - (int64_t)a.r * a.Sq;
            }
        };
        // row statistics of the prefetched rows into stage `stage`; dSinks terms of own rows
        auto statistics = [&](const WinPos &pos, int stage) __attribute__((always_inline)) {
            typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    union { uint32_t u; bf16x2 v; } x, y;
                    x.u = pre_o[j][e];
                    y.u = pre_g[j][e];
                    acc = __builtin_amdgcn_fdot2_f32_bf16(x.v, y.v, acc, false);
                }
            acc += __shfl_xor(acc, 1);
            const float lse2 = pre_lse * kLog2e;
            if (hr == 0) {
                sstat[(stage * 2 + 0) * kTile + srow] = lse2;
                sstat[(stage * 2 + 1) * kTile + srow] = -acc;
            }
            if (a.dsinks && pos.t < t1) {                       // rows of the chunk itself, each counted once
                const float sink2 = (sinks ? sinks[g * a.r + pos.h] : 0.0f) * kLog2e;
                const float term = (hr == 0 && pos.t * kTile + srow < a.Sq) ? fast_exp2(sink2 - lse2) * -acc : 0.0f;
                my_sink[pos.h * 64] += term;
            }
        };

        WinPos p_stat{t0, 0}, p_pre{t0, 0}, p_prev{t0, 0};
        prefetch(p_pre);
        wait_vmcnt<0>();
        __syncthreads();                                       // the K slabs are in LDS
        // K^T fragments (A operands: lane = column, slots = keys) of the three live key tiles
        bf16x8 kfr[3][4][2];
#pragma unroll
        for (int p = 0; p < 3; ++p)
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int db = 0; db < 2; ++db) kfr[p][kk][db] = ofrag_tr(ds_base + p * kStageTileBytes, lo, kk >> 1, kk & 1, db);
        statistics(p_stat, 0);                                 // statistics of the first tile
        p_stat.step(a.r);
        if (n_it > 1) prefetch(p_pre);

        // dQ rows 32*hh.. of the tile at `pos` from the dS tile at LDS address ds_tile
        auto helper_dq = [&](uint32_t ds_tile, const WinPos &pos) __attribute__((always_inline)) {
            f32x16 acc[2];
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[db][i] = 0.0f;
#pragma unroll
            for (int p = 0; p < 3; ++p)
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    const bf16x8 ads = ofrag_tr(ds_tile + p * kStageTileBytes, lo, kk >> 1, kk & 1, hh);
#pragma unroll
                    for (int db = 0; db < 2; ++db) acc[db] = mfma_bf16(kfr[p][kk][db], ads, acc[db]);
                }
            const int r0 = pos.t * kTile + 32 * hh;
            const int head = g * a.r + pos.h;
            bf16 *row0 = a.dq + (int64_t)b * a.dqs.b + (int64_t)head * a.dqs.h + (int64_t)r0 * a.dqs.s;
            store_rows32(out_stage, acc, a.scale, row0, a.dqs.s, a.Sq - r0, lane);
            __builtin_amdgcn_wave_barrier();
        };
        auto reload = [&](auto slot_tag) __attribute__((always_inline)) {
            constexpr int P = decltype(slot_tag)::value;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int db = 0; db < 2; ++db) kfr[P][kk][db] = ofrag_tr(transit_base, lo, kk >> 1, kk & 1, db);
        };

        WinPos cur{t0, 0};
        for (int it = 0; it < n_it; ++it) {
            __syncthreads();
            if (it > 0 && p_prev.t < t1) helper_dq(ds_base + ((it - 1) & 1) * C::kDsBytes, p_prev);
            if (cur.h == 0 && cur.t > t0 && cur.t < t1) {
                // key tile cur.t has arrived in the transit buffer; it replaces tile cur.t - 3
                const int slot = cur.t % 3;
                if (slot == 0) reload(std::integral_constant<int, 0>{});
                else if (slot == 1) reload(std::integral_constant<int, 1>{});
                else reload(std::integral_constant<int, 2>{});
            }
            if (it + 1 < n_it) {
                statistics(p_stat, (it + 1) % NS);
                p_stat.step(a.r);
            }
            if (it + 2 < n_it) prefetch(p_pre);
            p_prev = cur;
            cur.step(a.r);
        }
        __syncthreads();                                       // the last dS tile is complete
        if (p_prev.t < t1) helper_dq(ds_base + ((n_it - 1) & 1) * C::kDsBytes, p_prev);
        if (a.dsinks) {
            for (int h = 0; h < a.r; ++h) {
                float v = my_sink[h * 64];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
                if (lane == 0) a.dsink_partial[((((int64_t)b * n_chunks + chunk) * a.G + g) * a.r + h) * C::NHELP + hh] = v;
            }
        }
        return;
    }

    // ===================================== owner wavefronts =====================================
    const int pair = w >> 1, sub = w & 1;
    int my_kt = tile_of_slot(pair, t0);                        // key tile held (negative: none yet)
    bf16x8 kf[1][4], vf[1][4];
    f32x16 dk[1][2], dv[1][2];
    auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 16; ++i) { dk[0][0][i] = dk[0][1][i] = 0.0f; dv[0][0][i] = dv[0][1][i] = 0.0f; }
    };
    {
        const int j = my_kt * kTile + 32 * sub + l32;
        const bool ok = my_kt >= 0 && j < a.Skv;
        const bf16 *krow = kbase + (int64_t)(ok ? j : 0) * a.ks.s;
        const bf16 *vrow = vbase + (int64_t)(ok ? j : 0) * a.vs.s;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            u32x4 zk = {0u, 0u, 0u, 0u}, zv = {0u, 0u, 0u, 0u};
            if (ok) {
                zk = *reinterpret_cast<const u32x4 *>(krow + 16 * ks + 8 * half);
                zv = *reinterpret_cast<const u32x4 *>(vrow + 16 * ks + 8 * half);
            }
            kf[0][ks] = as_bf16x8(zk);
            vf[0][ks] = as_bf16x8(zv);
        }
        clear_acc();
    }
    // dK / dV of the key tile held, if it is one of the chunk's own
    // fp32 share of a seam tile: [b][g][seam][tile 0/1][workgroup before / after the seam][dK, dV][64 keys][64]
    auto seam_slot = [&](int seam, int tile, int side) {
        return a.boundary_partial + (((((int64_t)b * a.G + g) * (n_chunks - 1) + seam) * 2 + tile) * 2 + side) * (2 * kTile * kD);
    };
    auto store_share = [&](float *dst) __attribute__((always_inline)) {
        // unscaled fp32 sums; lane = key row, register i of block dblk = column 32*dblk + crow(i, half),
        // four consecutive columns per 16-byte store
        float *pk = dst + (32 * sub + l32) * kD, *pv = pk + kTile * kD;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const int col = 32 * dblk + 8 * a4 + 4 * half;
                f32x4 xk, xv;
#pragma unroll
                for (int e = 0; e < 4; ++e) { xk[e] = dk[0][dblk][4 * a4 + e]; xv[e] = dv[0][dblk][4 * a4 + e]; }
                *reinterpret_cast<f32x4 *>(pk + col) = xk;
                *reinterpret_cast<f32x4 *>(pv + col) = xv;
            }
    };
    // dK / dV of the key tile held: written out if it is complete, left as this workgroup's share if
    // it sits on a seam, dropped if it belongs to the neighbour (recomputation mode)
    auto flush = [&]() __attribute__((always_inline)) {
        if (my_kt < 0) return;
        if (seam_sums) {
            if (my_kt < t0) { store_share(seam_slot(chunk - 1, my_kt - (t0 - 2), 1)); return; }
            if (my_kt >= t1 - 2 && t1 < nT) { store_share(seam_slot(chunk, my_kt - (t1 - 2), 0)); return; }
        } else if (my_kt < t0 || my_kt >= t1) {
            return;
        }
        const int r0 = my_kt * kTile + 32 * sub;
        const int nvalid = a.Skv - r0;
        store_rows32(out_stage, dk[0], a.scale, a.dk + (int64_t)b * a.dks.b + (int64_t)g * a.dks.h + (int64_t)r0 * a.dks.s,
                     a.dks.s, nvalid, lane);
        __builtin_amdgcn_wave_barrier();
        store_rows32(out_stage, dv[0], 1.0f, a.dv + (int64_t)b * a.dvs.b + (int64_t)g * a.dvs.h + (int64_t)r0 * a.dvs.s,
                     a.dvs.s, nvalid, lane);
        __builtin_amdgcn_wave_barrier();
    };

    const float c = a.scale_log2;
    int dead[1] = {0};
    const uint32_t ds_out0 = ds_store_addr(ds_base + pair * kStageTileBytes, 32 * sub + l32, half);

    // ---- copies: wavefront kWaveQ the Q tile, wavefront kWaveDO the dO tile of each walk position (eight
    // 16-byte-per-lane instructions), wavefront kWaveTransit the K and V rows of the next key tile ----
    constexpr int kWaveQ = 2, kWaveDO = 3, kWaveTransit = 0;   // the copying owners share their SIMDs with the (lighter) helpers
    const int64_t lstride = (w == kWaveQ) ? a.qs.s : a.dos.s;
    const int64_t ld_hstride = (w == kWaveQ) ? a.qs.h : a.dos.h;
    uint32_t ld_off[2];
    {
        const int lr = lane >> 3;
        ld_off[0] = (uint32_t)(lr * (int)lstride + (((lane & 7) ^ swz(lr)) * 8));
        ld_off[1] = (uint32_t)(lr * (int)lstride + (((lane & 7) ^ swz(lr + 8)) * 8));
    }
    int iss_h = 0, iss_i0 = t0 * kTile;
    const bf16 *ld_tile = (w == kWaveQ)
        ? a.q + (int64_t)b * a.qs.b + (int64_t)(g * a.r) * a.qs.h + (int64_t)iss_i0 * a.qs.s
        : a.d_o + (int64_t)b * a.dos.b + (int64_t)(g * a.r) * a.dos.h + (int64_t)iss_i0 * a.dos.s;
    auto issue = [&](int it) __attribute__((always_inline)) {
        const int stage = it % NS;
        if (w == kWaveQ || w == kWaveDO) {
            char *dst = smem + (stage * 2 + (w - kWaveQ)) * kStageTileBytes;
            if (iss_i0 + kTile <= a.Sq) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(ld_tile + (int64_t)(8 * k) * lstride + ld_off[k & 1]),
                                                     (lds_void_t *)(dst + 8 * k * kRowBytes), 16, 0, 0);
            } else {
                // the tile sticks out of the tensor: rows past the end re-read the last valid one
                // (rare: a rolled loop keeps its address arithmetic out of the registers of the main loop)
#pragma unroll 1
                for (int k = 0; k < 8; ++k) {
                    const int rr = 8 * k + (lane >> 3);
                    const int cc = (lane & 7) ^ swz(rr);
                    const int over = max(0, iss_i0 + rr - (a.Sq - 1));
                    __builtin_amdgcn_global_load_lds((glb_void_t *)(ld_tile + (int64_t)(rr - over) * lstride + cc * 8),
                                                     (lds_void_t *)(dst + 8 * k * kRowBytes), 16, 0, 0);
                }
            }
        }
        ++iss_h;
        ld_tile += ld_hstride;
        if (iss_h == a.r) {
            iss_h = 0;
            iss_i0 += kTile;
            ld_tile += (int64_t)kTile * lstride - (int64_t)a.r * ld_hstride;
        }
    };
    auto issue_transit = [&](int kt) __attribute__((always_inline)) {
#pragma unroll 1
        for (int k = 0; k < 8; ++k) {
            const int rr = 8 * k + (lane >> 3);
            const int cc = (lane & 7) ^ swz(rr);
            const int row = min(kt * kTile + rr, a.Skv - 1);
            __builtin_amdgcn_global_load_lds((glb_void_t *)(kbase + (int64_t)row * a.ks.s + cc * 8),
                                             (lds_void_t *)(transit + 8 * k * kRowBytes), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_void_t *)(vbase + (int64_t)row * a.vs.s + cc * 8),
                                             (lds_void_t *)(transit + kStageTileBytes + 8 * k * kRowBytes), 16, 0, 0);
        }
    };

    wait_vmcnt<0>();
    __syncthreads();                                           // prologue barrier (the helpers read the K slabs now)
    issue(0);
    if (n_it > 1) issue(1);

    WinPos cur{t0, 0};
    // One copy of the loop body with the LDS stage as a run-time value: a body per stage (stage
    // offsets as instruction immediates) makes this kernel larger than the instruction cache.
    int stage = 0;
    // the fragment offsets with the address of the stage at hand folded in: one add each per walk position, and every
    // read of the position's Q and dO tiles is (register) + (immediate)
    TileLaneOffsets lo_st = tile_offsets_at(lo, smem_base);
    uint32_t lo_st_at = smem_base;
    auto iterate = [&](int it) __attribute__((always_inline)) {
        const int STAGE = stage;
        stage = stage == NS - 1 ? 0 : stage + 1;
        {
            const uint32_t at = smem_base + STAGE * (2 * kStageTileBytes);
            tile_offsets_move(lo_st, at - lo_st_at);
            lo_st_at = at;
        }
        if (w == kWaveQ || w == kWaveDO) { if (it + 1 >= n_it) wait_vmcnt<0>(); else wait_vmcnt<8>(); }
        else if (w == kWaveTransit && cur.h == 0) wait_vmcnt<0>();        // the transit copy of the key tile that starts now
        __syncthreads();
        if (it + 2 < n_it) issue(it + 2);
        if (w == kWaveTransit && cur.h == 1 && cur.t + 1 < t1) issue_transit(cur.t + 1);

        if (cur.h == 0 && cur.t > t0 && pair == cur.t % 3) {
            // this pair's key tile (cur.t - 3) is complete; take over key tile cur.t from the transit buffer
            flush();
            my_kt = cur.t < t1 ? cur.t : -1;
            if (my_kt >= 0) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    kf[0][ks] = ofrag_nat(transit_base - lo_st_at, lo_st, sub, ks);
                    vf[0][ks] = ofrag_nat(transit_base + kStageTileBytes - lo_st_at, lo_st, sub, ks);
                }
            }
            clear_acc();
        }

        const int i0 = cur.t * kTile;
        const uint32_t ds_out = ds_out0 + (it & 1) * C::kDsBytes;
        const int wj0 = my_kt * kTile + 32 * sub;              // first key of the wavefront
        const int pos0 = i0;
        const int pos1 = min(min(a.Sq, i0 + kTile) - 1, q_len - 1);
        const int wj1 = min(wj0 + 32, kv_len) - 1;
        const bool skip = my_kt < 0 || wj1 < wj0 || pos1 < wj0 || pos0 > wj1 + weff - 1 || pos1 < pos0;
        if (skip) {
            ds_store_zero(ds_out, 0);
            ds_store_zero(ds_out, 1);
        } else {
            // (fragment addresses: the stage's address is in the lane offsets, the dO tile is 8 KB behind Q's)
            const uint32_t qsm = 0u, gsm = kStageTileBytes;
            const uint32_t stat_lane = stat_base + STAGE * (2 * kTile * 4) + half * 16;
            const bool interior = (wj0 + 31 <= pos0) && (wj0 > pos1 - weff) && (wj0 + 32 <= kv_len) && (i0 + kTile - 1 <= pos1);
            int jkey[1] = {wj0 + l32};
            if (interior) {
                dkdv_tile<false, false, 1, true>(qsm, gsm, stat_lane, lo_st, kf, vf, dk, dv, c, half, dead, 0u, 0, 0, 0u, jkey, ds_out);
            } else {
                int dbase[1];
                dbase[0] = (wj0 + l32 < kv_len) ? pos0 - (wj0 + l32) : -0x40000000;
                const int row_lim = min(kTile, min(a.Sq, q_len) - i0);
                dkdv_tile<true, false, 1, true>(qsm, gsm, stat_lane, lo_st, kf, vf, dk, dv, c, half, dbase, (unsigned)weff, row_lim,
                                                wj0 - pos0, 0u, jkey, ds_out);
            }
        }
        cur.step(a.r);
    };

    for (int it = 0; it < n_it; ++it) iterate(it);
    __syncthreads();                                           // hands the last dS tile over
    flush();
}

// ---------------------------------------------------------------------------------
// What is left after the window kernel, in one small launch.  Blocks [0, seam_blocks): dK / dV of
// the seam tiles = round(scale * (share of the workgroup before the seam + share of the one after)),
// one thread per 16-byte output chunk.  Blocks from seam_blocks on: one block per query head adds
// that head's dSinks partial sums (per batch row, chunk and helper) in a fixed tree order.
__global__ __launch_bounds__(256) void attn_bwd_window_finish_kernel(const KArgs a, int n_chunks, int seam_blocks) {
    if ((int)blockIdx.x >= seam_blocks) {
        __shared__ float red[256];
        const int h = blockIdx.x - seam_blocks;
        const int n = a.B * n_chunks * WinCfg::NHELP;
        float acc = 0.0f;
        for (int i = threadIdx.x; i < n; i += 256) {
            const int bc = i / WinCfg::NHELP, e = i % WinCfg::NHELP;
            acc += a.dsink_partial[((int64_t)bc * a.H + h) * WinCfg::NHELP + e];
        }
        red[threadIdx.x] = acc;
        __syncthreads();
        for (int off = 128; off > 0; off >>= 1) {
            if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
            __syncthreads();
        }
        if (threadIdx.x == 0) a.dsinks[h] = red[0];
        return;
    }
    // chunk index over (b, g, seam, tile, tensor, key, 8 columns)
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int c8 = (int)(idx & 7) * 8;
    const int key = (int)((idx >> 3) & 63);
    const int which = (int)((idx >> 9) & 1);                      // 0 = dK, 1 = dV
    const int tile = (int)((idx >> 10) & 1);
    const int64_t rest = idx >> 11;                               // (b * G + g) * (n_chunks - 1) + seam
    if (rest >= (int64_t)a.B * a.G * (n_chunks - 1)) return;
    const int seam = (int)(rest % (n_chunks - 1));
    const int bg = (int)(rest / (n_chunks - 1));
    const int g = bg % a.G, b = bg / a.G;
    const int row = ((seam + 1) * a.chunk_tiles - 2 + tile) * kTile + key;
    if (row >= a.Skv) return;
    const float *before = a.boundary_partial + ((rest * 2 + tile) * 2 + 0) * (2 * kTile * kD) + (which * kTile + key) * kD + c8;
    const float *after = before + 2 * kTile * kD;
    const float mul = which == 0 ? a.scale : 1.0f;
    bf16x8 out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const f32x4 x = *reinterpret_cast<const f32x4 *>(before + 4 * j), y = *reinterpret_cast<const f32x4 *>(after + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; ++e) out[4 * j + e] = (bf16)((x[e] + y[e]) * mul);
    }
    const Strides &st = which == 0 ? a.dks : a.dvs;
    bf16 *dst = (which == 0 ? a.dk : a.dv) + (int64_t)b * st.b + (int64_t)g * st.h + (int64_t)row * st.s + c8;
    union { bf16x8 v; u32x4 u; } cv;
    cv.v = out;
    *reinterpret_cast<u32x4 *>(dst) = cv.u;
}

}  // namespace gptoss
