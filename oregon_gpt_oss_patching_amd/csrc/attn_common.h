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
constexpr int kLS = 72;         // LDS row stride in elements (64 + 8 pad: 16-byte
                                // reads of 8 consecutive rows fall in distinct banks)
constexpr int kTileElems = kTile * kLS;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Strides { int64_t b, h, s; };

struct KArgs {
    const bf16 *q, *k, *v;
    const float *sinks;
    const int32_t *seqlens;
    bf16 *o;
    float *lse;
    const bf16 *d_o;
    bf16 *dq, *dk, *dv;
    float *dsinks;
    float *delta;
    Strides qs, ks, vs, os, dos, dqs, dks, dvs;
    int B, H, G, Sq, Skv;
    int r;               // H / G query heads per KV head
    int window;          // 0 = full causal
    int q_offset;
    float scale;
    float scale_log2;    // scale * log2(e)
};

__device__ __forceinline__ int crow(int i, int half) { return 8 * (i >> 2) + 4 * half + (i & 3); }

__device__ __forceinline__ f32x16 mfma_bf16(const bf16x8 a, const bf16x8 b, const f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 as_bf16x8(const u32x4 v) {
    union { u32x4 u; bf16x8 b; } x; x.u = v; return x.b;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- staging a 64 x 64 tile: global -> registers -> LDS, NT threads --------------
// Thread t owns 16-byte chunk (t % 8) of rows (t / 8) + k * (NT / 8): eight
// consecutive lanes read one whole 128-byte row, so global loads are fully
// coalesced 128-bit accesses and the LDS writes of a row are contiguous.
template <int NT>
struct TileRegs { u32x4 v[512 / NT]; };

template <int NT>
__device__ __forceinline__ void tile_load(TileRegs<NT> &r, const bf16 *base, int64_t stride_s,
                                          int row0, int row_end, int tid) {
    const int c = tid & 7, rr = tid >> 3;
#pragma unroll
    for (int pass = 0; pass < 512 / NT; ++pass) {
        const int row = row0 + rr + (NT / 8) * pass;
        u32x4 z = {0u, 0u, 0u, 0u};
        if (row < row_end) z = *reinterpret_cast<const u32x4 *>(base + (int64_t)row * stride_s + c * 8);
        r.v[pass] = z;
    }
}

template <int NT>
__device__ __forceinline__ void tile_store(bf16 *lds, const TileRegs<NT> &r, int tid) {
    const int c = tid & 7, rr = tid >> 3;
#pragma unroll
    for (int pass = 0; pass < 512 / NT; ++pass)
        *reinterpret_cast<u32x4 *>(lds + (rr + (NT / 8) * pass) * kLS + c * 8) = r.v[pass];
}

// A (or B) fragment with the contraction along head_dim: lane reads
// tile[32*blk + l32][16*ks + 8*half .. +8], one 128-bit LDS read.
__device__ __forceinline__ bf16x8 frag_nat(const bf16 *lds, int blk, int ks, int lane) {
    const int row = 32 * blk + (lane & 31), col = 16 * ks + 8 * (lane >> 5);
    return as_bf16x8(*reinterpret_cast<const u32x4 *>(lds + row * kLS + col));
}

// A fragment of the TRANSPOSED tile, contraction along the tile's rows:
// lane ends up holding tile[rows(half, slot)][32*dblk + l32] for slots 0..7 with
//   rows(half, 4*t + e) = 32*blk + 16*u + 8*t + 4*half + e  = 32*blk + crow(8*u + 4*t + e, half),
// i.e. exactly the rows that C registers 8*u .. 8*u+7 of row-block `blk` hold, so
// those registers (converted to bf16) are the matching B fragment.
// ds_read_b64_tr_b16 semantics (within each group of 16 lanes, i = lane % 16):
//   result[i][e] = chunk[lane 4*e + i/4][i % 4], chunk[j] = the 4 halfwords at lane j's address.
// Lane j therefore points at row (base + j/4), columns (dg + 4*(j%4)) .. +3.
__device__ __forceinline__ bf16x8 frag_tr(const bf16 *lds, int blk, int u, int dblk, int lane) {
    const int i = lane & 15, g16 = lane >> 4, half = g16 >> 1;
    const int col = 32 * dblk + 16 * (g16 & 1) + 4 * (i & 3);
    const int row = 32 * blk + 16 * u + 4 * half + (i >> 2);
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const bf16 *p0 = lds + row * kLS + col;
    const bf16 *p1 = p0 + 8 * kLS;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p1));
    union { struct { s16x4 a, b; } s; bf16x8 v; } x;
    x.s.a = lo; x.s.b = hi;
    return x.v;
}

// B fragment from C registers 8*u .. 8*u+7 (see frag_tr).
__device__ __forceinline__ bf16x8 cfrag(const f32x16 &c, int u) {
    bf16x8 f;
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (bf16)c[8 * u + j];
    return f;
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
