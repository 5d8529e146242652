// Shared device helpers for the gfx950 GPT-OSS attention kernels: vector types,
// MFMA wrappers and the LDS tile layout every kernel stages K/V/Q/dO through.
//
// Register layouts of v_mfma_f32_32x32x16_bf16 used throughout (lane = 0..63,
// half = lane / 32, l32 = lane % 32):
//   A (32 x 16): lane holds A[l32][8*half + 0..7]
//   B (16 x 32): lane holds B[8*half + 0..7][l32]
//   C (32 x 32): register i holds C[crow(i, half)][l32],
//                crow(i, half) = 8*(i/4) + 4*half + i%4
// Because the k-slot -> contraction-index mapping is the same for A and B, any
// consistent choice of which real index sits in slot (half, j) is legal; the
// kernels exploit this to feed C registers straight back in as a B operand.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gptoss {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int kD = 64;          // head_dim handled by these kernels
constexpr int kTile = 64;       // rows per staged LDS tile
constexpr int kLS = 72;         // row stride (elements) of the padded output stage (64 + 8 pad: 16-byte
                                // reads of 8 consecutive rows fall in distinct banks)
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Strides { int64_t b, h, s; };

struct KArgs {
    const bf16 *q, *k, *v;
    const float *sinks;
    const int32_t *seqlens;
    const int32_t *doc_start;   // optional (B, Sq): first key of each query's document
    bf16 *o;
    float *lse;
    const bf16 *d_o;
    bf16 *dq, *dk, *dv;
    float *dsinks;
    float *delta;        // row statistics in fp32: -delta[B][H][Sq], then lse * log2(e) [B][H][Sq]
    u32x4 *split;        // the same statistics as bf16 triples, 16 bytes per row (see split_row_stats)
    Strides qs, ks, vs, os, dos, dqs, dks, dvs;
    int B, H, G, Sq, Skv;
    int r;               // H / G query heads per KV head
    int window;          // 0 = full causal
    int q_offset;
    const int32_t *q_offset_dev;  // if set, the offset is read from device memory and q_offset is ignored
    float scale;
    float scale_log2;    // scale * log2(e)
    int dkdv_parts;      // dK/dV kernel: workgroups that share one key block, each taking a slice of its query tiles
    float *dkdv_partial; // dkdv_parts > 1: fp32 partial sums, [part][dK, dV][B][G][Skv][64]
    int chunk_tiles;     // single-pass window backward: 64-row query tiles per workgroup
    float *dsink_partial; // single-pass window backward: dSinks partial sums, [B][chunk][H][2]
    float *boundary_partial; // single-pass window backward: fp32 dK / dV shares of the tiles on chunk seams, or NULL
};

// Absolute position of query row 0: by value, or (for callers that must not synchronise with the
// device to learn it) from device memory, one scalar load per workgroup.
__device__ __forceinline__ int query_offset(const KArgs &a) {
    if (!a.q_offset_dev) return a.q_offset;
    const int v = __builtin_amdgcn_readfirstlane(*a.q_offset_dev);
    return min(max(v, 0), (1 << 30) - a.Sq);      // what the host checks for an offset passed by value
}


__device__ __forceinline__ int crow(int i, int half) { return 8 * (i >> 2) + 4 * half + (i & 3); }

__device__ __forceinline__ f32x16 mfma_bf16(const bf16x8 a, const bf16x8 b, const f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 as_bf16x8(const u32x4 v) {
    union { u32x4 u; bf16x8 b; } x; x.u = v; return x.b;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- row statistics as an MFMA operand -----------------------------------------------------------
// The dK/dV kernels need, for every element of a 32 x 32 block of S and dP, a number that belongs to the
// element's ROW (lse and delta), while a lane of the MFMA result holds one COLUMN: read as they are, the
// statistics cost eight broadcast LDS reads per block.  Instead they enter through the matrix pipe as one
// more step of the contraction: the A operand of that step holds, per row, L = lse / scale and -delta, each
// split into three bf16 terms whose sum is the fp32 value (3 x 8 mantissa bits; the products with +-1 are
// exact and the accumulation is fp32), and the B operand holds -1 against the terms of L (for S) or +1
// against the terms of -delta (for dP), so that the MFMAs deliver S - L and dP - delta and
// P = exp2((S - L) * scale * log2(e)).
//   row layout (8 bf16): L_hi, L_mid, L_lo, 0, nd_hi, nd_mid, nd_lo, 0
__device__ __forceinline__ void split3_bf16(float x, uint32_t &w01, uint32_t &w2) {
    union { bf16 h; uint16_t u; } hi, mid, lo;
    hi.h = (bf16)x;
    const float r1 = x - (float)hi.h;       // exact
    mid.h = (bf16)r1;
    const float r2 = r1 - (float)mid.h;     // exact
    lo.h = (bf16)r2;
    w01 = (uint32_t)hi.u | ((uint32_t)mid.u << 16);
    w2 = (uint32_t)lo.u;
}
__device__ __forceinline__ u32x4 split_row_stats(float lse, float scale, float neg_delta) {
    uint32_t w0, w1, w2, w3;
    split3_bf16(lse / scale, w0, w1);
    split3_bf16(neg_delta, w2, w3);
    return u32x4{w0, w1, w2, w3};
}
// B operands of the statistics step; only the lanes of half 0 carry k = 0..7 of the 16-deep step, and the
// A operand repeats the row's 16 bytes in both halves (finite times zero)
__device__ __forceinline__ void stat_step_operands(int half, bf16x8 &b_s, bf16x8 &b_dp) {
    const u32x4 s = {half ? 0u : 0xBF80BF80u, half ? 0u : 0x0000BF80u, 0u, 0u};
    const u32x4 d = {0u, 0u, half ? 0u : 0x3F803F80u, half ? 0u : 0x00003F80u};
    b_s = as_bf16x8(s);
    b_dp = as_bf16x8(d);
}
// max(a, b) as median(a, b, +inf): one v_med3_f32, without the NaN-quieting pre-pass that
// fmaxf costs in IEEE mode (the kernels never produce NaN: masked logits are -inf and the
// running max is finite).
__device__ __forceinline__ float fast_max(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, INFINITY); }
// max(x of this lane, x of lane ^ 32): v_permlane32_swap exchanges the two 32-lane halves in
// the VALU, so the reduction does not queue behind outstanding LDS reads as a ds_bpermute would.
// swap(a, b) returns {a.lo | b.lo, a.hi | b.hi} (low 32 lanes | high 32 lanes).
__device__ __forceinline__ float xhalf_max(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
    const unsigned u = __float_as_uint(x);
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned lo = r.x, hi = r.y;     // copied out first: bit-casting the vector elements in place reads element 0 twice
    return fast_max(__uint_as_float(lo), __uint_as_float(hi));
}
// x of this lane + x of lane ^ 32 (same exchange as xhalf_max)
__device__ __forceinline__ float xhalf_sum(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
    const unsigned u = __float_as_uint(x);
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const unsigned lo = r.x, hi = r.y;
    return __uint_as_float(lo) + __uint_as_float(hi);
}
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Visibility test of the kernels whose lanes are query rows and whose accumulator registers are
// keys (forward, dQ).  Key r of the tile is visible to the lane iff 0 <= dbase - r < wl and
// r < key_lim, where dbase = (lane's query position) - (first key of the tile), hugely negative
// for a dead row.  Register i of a 32-key block holds key r = rc + 4*half with rc a compile-time
// constant, so with everything lane-dependent folded into two values per tile the test is
// (unsigned)(base - rc) < width: one subtract, one compare, one select per element.
struct KeyMask { int base; unsigned width; };
__device__ __forceinline__ KeyMask make_key_mask(int dbase, unsigned wl, int key_lim, int half) {
    const int dbh = dbase - 4 * half;
    const int kl = min(max(key_lim, -8), 72) - 4 * half;     // only its relation to 0..63 matters
    const int lo = max(0, dbh - kl + 1);                       // dbase - r >= lo  <=>  r < key_lim (and r <= dbase)
    KeyMask m;
    m.base = dbh - lo;
    m.width = (unsigned)max(0, (int)wl - lo);
    return m;
}
__device__ __forceinline__ bool key_visible(const KeyMask &m, int rc) { return (unsigned)(m.base - rc) < m.width; }

// B fragment from C registers 8*u .. 8*u+7: converted to bf16 they hold, in k-slot order, exactly
// the rows that a transposed A fragment (ofrag_tr) of the same 16-row step holds.
__device__ __forceinline__ bf16x8 cfrag(const f32x16 &c, int u) {
    bf16x8 f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (bf16)c[8 * u + j];
    return f;
}

// ---- asynchronous tile staging: global -> LDS without passing through registers ----
// global_load_lds_dwordx4 writes lane L's 16 bytes at (wave-uniform LDS base) + 16*L,
// so one instruction fills 8 unpadded 128-byte rows.  To keep the later fragment reads
// free of bank conflicts the 16-byte chunks of a row are XOR-swizzled: physical chunk p
// of tile row r holds logical chunk p ^ swz(r).  swz() is chosen so that
//   * 16 consecutive rows reading the same logical chunk (natural 128-bit fragment
//     reads) fall in 16 distinct 16-byte bank groups, and
//   * 4 consecutive rows x 2 adjacent chunks (transposing 64-bit reads) do as well.
constexpr int kRowBytes = kD * 2;                 // 128
constexpr int kStageTileBytes = kTile * kRowBytes; // 8192

__device__ __forceinline__ int swz(int r) { return (((r >> 1) & 1) << 2) | (((r >> 3) & 1) << 1) | ((r >> 2) & 1); }

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

// The copy instruction written as inline assembly (used by the hand-pipelined kernels, attn_bwd_dkdv64_kernel
// and attn_fwd_pipe_kernel).  Issued through
// the compiler's builtin, every LDS read that follows a copy is made to wait for ALL outstanding copies (the
// compiler cannot tell which LDS bytes a copy writes, and a workgroup barrier waits for them as well), which
// turns a three-stage pipeline into "issue, wait for what was just issued, compute".  Hidden in the
// assembly the copies are invisible to that bookkeeping; ordering is then entirely the kernel's
// business: wait_vmcnt<N>() before the barrier that hands a stage to its readers, and a barrier
// between the last read of a stage and the copy that overwrites it.  (Compiler-generated vmcnt waits
// for its own loads stay correct: loads return in order, so unknown extra loads only make such a wait
// longer.)  M0 holds the wave-uniform LDS base; nothing else in these kernels uses M0.  The kernels whose key
// loops are scheduled by the compiler (attn_fwd_kernel, attn_bwd_dq_kernel) keep the builtin: their wavefronts
// alternate between stretches of MFMAs and stretches of vector work whatever the copies do, and the hidden
// form measured the same or slower there.
// lane L's 16 bytes at gbase + voff land at lds_base + 16 * L
__device__ __forceinline__ void lds_dma16(uint32_t lds_base, const void *gbase, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(gbase) : "memory");
}
// the same with the LDS base given as (scalar register) + (compile-time constant): one scalar instruction
// forms the sum in M0
template <int IMM>
__device__ __forceinline__ void lds_dma16_plus(uint32_t lds_base, const void *gbase, uint32_t voff) {
    if constexpr (IMM == 0) lds_dma16(lds_base, gbase, voff);
    else asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voff), "s"(gbase), "n"(IMM) : "memory", "scc");
}
// lane L's 4 bytes at gbase + voff land at lds_base + 4 * L
__device__ __forceinline__ void lds_dma4(uint32_t lds_base, const void *gbase, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_base), "v"(voff), "s"(gbase) : "memory");
}
// the same with the LDS base given as the sum of two scalar registers, formed in M0 by one instruction
__device__ __forceinline__ void lds_dma4_at(uint32_t lds_base, uint32_t lds_off, const void *gbase, uint32_t voff) {
    asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3" ::"s"(lds_base), "s"(lds_off), "v"(voff), "s"(gbase) : "memory", "scc");
}

// Issues the 4-wavefront asynchronous copy of tile rows [row0, row0+64) (rows at or
// beyond row_end re-read the last valid row: their products are masked, they only
// have to be finite).  Each wavefront issues two instructions.
__device__ __forceinline__ void tile_async(char *lds_tile, const bf16 *base, int64_t stride_s, int row0,
                                           int row_end, int lane, int w) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int r = 16 * w + 8 * k + (lane >> 3);
        const int c = (lane & 7) ^ swz(r);
        const int row = min(row0 + r, row_end - 1);
        const bf16 *src = base + (int64_t)row * stride_s + c * 8;
        __builtin_amdgcn_global_load_lds((glb_void_t *)src, (lds_void_t *)(lds_tile + (16 * w + 8 * k) * kRowBytes), 16, 0, 0);
    }
}

// The same copy with the lane-dependent part of the address precomputed: lane offsets (in
// bytes, so that the address is exactly (scalar pointer) + (zero-extended 32-bit register), the
// form the instruction takes without any address arithmetic) of the wavefront's two 16-byte
// chunks relative to the tile's first row.  Only valid
// for tiles that lie completely inside the tensor (no row clamping); `tile` points at the
// tile's first row and is wave-uniform, so the loads use scalar base + 32-bit lane offset.
struct AsyncLaneOffsets { uint32_t off[2]; };

__device__ __forceinline__ AsyncLaneOffsets make_async_offsets(int64_t stride_s, int lane, int w) {
    AsyncLaneOffsets o;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int r = 16 * w + 8 * k + (lane >> 3);
        const int c = (lane & 7) ^ swz(r);
        o.off[k] = (uint32_t)(r * (int)stride_s + c * 8) * 2u;
    }
    return o;
}

__device__ __forceinline__ void tile_async_inner(char *lds_tile, const bf16 *tile, const AsyncLaneOffsets &o, int w) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        __builtin_amdgcn_global_load_lds((glb_void_t *)(reinterpret_cast<const char *>(tile) + o.off[k]),
                                         (lds_void_t *)(lds_tile + (16 * w + 8 * k) * kRowBytes), 16, 0, 0);
    }
}

// Waits until at most `n` of this wavefront's vector-memory operations are outstanding.
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// ---- register-cheap addressing of swizzled tiles --------------------------------
// All lane-dependent parts of the fragment addresses are computed once per kernel
// (TileLaneOffsets); inside the loops an address is (stage base + lane offset) with
// the block / tile selection folded into the instruction's immediate offset.
typedef __attribute__((address_space(3))) char lds_char_t;

__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(lds_char_t *)p;
}
__device__ __forceinline__ u32x4 lds_load128(uint32_t addr, int imm) {
    return *reinterpret_cast<const __attribute__((address_space(3))) u32x4 *>((uintptr_t)(addr + imm));
}
__device__ __forceinline__ f32x4 lds_load128f(uint32_t addr, int imm) {
    return *reinterpret_cast<const __attribute__((address_space(3))) f32x4 *>((uintptr_t)(addr + imm));
}
__device__ __forceinline__ s16x4 lds_load_tr64(uint32_t addr, int imm) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(uintptr_t)(addr + imm));
}

struct TileLaneOffsets {
    uint32_t nat[4];      // [ks]: natural fragment, row l32 of block 0
    uint32_t tr[2][2];    // [dblk][t]: transposed fragment, u = 0 of block 0, rows (+8*t)
};

__device__ __forceinline__ TileLaneOffsets make_tile_offsets(int lane) {
    TileLaneOffsets o;
    {
        const int row = lane & 31;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) o.nat[ks] = row * kRowBytes + (((2 * ks + (lane >> 5)) ^ swz(row)) * 16);
    }
    {
        const int i = lane & 15, g16 = lane >> 4, half = g16 >> 1;
        const int sub = (i & 1) * 8;
#pragma unroll
        for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int row = 4 * half + (i >> 2) + 8 * t;
                const int chunk = 4 * dblk + 2 * (g16 & 1) + ((i & 3) >> 1);
                o.tr[dblk][t] = row * kRowBytes + ((chunk ^ swz(row)) * 16) + sub;
            }
    }
    return o;
}

// The lane offsets with a tile's (run-time) LDS address added once, for code that reads many fragments of one tile:
// the fragment reads then take (this register) + (immediate) and tile = 0.  The sums are hidden from the compiler,
// which otherwise folds the block / tensor constants into the scalar tile address and pays one vector add per read.
__device__ __forceinline__ TileLaneOffsets tile_offsets_at(const TileLaneOffsets &o, uint32_t tile) {
    TileLaneOffsets r;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) { r.nat[ks] = tile + o.nat[ks]; asm volatile("" : "+v"(r.nat[ks])); }
#pragma unroll
    for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
        for (int t = 0; t < 2; ++t) { r.tr[dblk][t] = tile + o.tr[dblk][t]; asm volatile("" : "+v"(r.tr[dblk][t])); }
    return r;
}

// moves such offsets from one tile address to another (delta = new address - old address, modulo 2^32)
__device__ __forceinline__ void tile_offsets_move(TileLaneOffsets &r, uint32_t delta) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) { r.nat[ks] += delta; asm volatile("" : "+v"(r.nat[ks])); }
#pragma unroll
    for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
        for (int t = 0; t < 2; ++t) { r.tr[dblk][t] += delta; asm volatile("" : "+v"(r.tr[dblk][t])); }
}

// natural fragment of 32-row block `blk`; `tile` = LDS byte address of the tile
__device__ __forceinline__ bf16x8 ofrag_nat(uint32_t tile, const TileLaneOffsets &o, int blk, int ks) {
    return as_bf16x8(lds_load128(tile + o.nat[ks], blk * 32 * kRowBytes));
}
// transposed fragment: rows 32*blk + 16*u + {4*half + 0..3, 8 + 4*half + 0..3}, columns 32*dblk + l32
__device__ __forceinline__ bf16x8 ofrag_tr(uint32_t tile, const TileLaneOffsets &o, int blk, int u, int dblk) {
    const int imm = (32 * blk + 16 * u) * kRowBytes;
    union { struct { s16x4 a, b; } s; bf16x8 v; } x;
    x.s.a = lds_load_tr64(tile + o.tr[dblk][0], imm);
    x.s.b = lds_load_tr64(tile + o.tr[dblk][1], imm);
    return x.v;
}

// Writes a wave's 32 x 64 result held as two transposed accumulators
// (lane = row l32, register i of acc[dblk] = column 32*dblk + crow(i, half)) to
// global memory through a wave-private LDS stage so that the global stores are
// whole 128-byte rows.  `stage` must hold 32 * kLS elements.
__device__ __forceinline__ void store_rows32(bf16 *stage, const f32x16 acc[2], float mul,
                                             bf16 *grow0, int64_t stride_s, int nvalid, int lane) {
    const int l32 = lane & 31, half = lane >> 5;
#pragma unroll
    for (int dblk = 0; dblk < 2; ++dblk)
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            bf16x4 pk;
#pragma unroll
            for (int e = 0; e < 4; ++e) pk[e] = (bf16)(acc[dblk][4 * a4 + e] * mul);
            *reinterpret_cast<bf16x4 *>(stage + l32 * kLS + 32 * dblk + 8 * a4 + 4 * half) = pk;
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int c = lane & 7, rr = lane >> 3;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int row = rr + 8 * pass;
        if (row < nvalid)
            *reinterpret_cast<u32x4 *>(grow0 + (int64_t)row * stride_s + c * 8) =
                *reinterpret_cast<const u32x4 *>(stage + row * kLS + c * 8);
    }
}

}  // namespace gptoss
