// Measurement aid, not part of the attention path: a loop of nothing but v_mfma_f32_32x32x16_bf16 on
// operands the caller supplies, two wavefronts per SIMD, four independent accumulators per wavefront.
// bench.py runs it on N(0,1) bf16 operands (and on zeros) to report what the matrix pipes of the part
// sustain on the contract's kind of data: under such a loop the clock is set by the power limit and
// depends on how many operand bits toggle, so the figure is well below the nominal peak and is the
// ceiling the attention kernels' executed MFMA rate can be compared with.
#pragma once
#include "attn_common.h"

namespace gptoss {

constexpr int kMfmaRateFrags = 4;              // A and B fragments per lane
constexpr int kMfmaRatePerIter = 4 * kMfmaRateFrags;   // MFMAs per loop pass and wavefront

// operands: n_vec 16-byte vectors (n_vec >= 1); lane t of the grid reads vectors (t * 8 + i) % n_vec
__global__ __launch_bounds__(256, 2) void mfma_rate_kernel(const u32x4 *operands, uint32_t n_vec, int iters, float *sink) {
    constexpr int NA = kMfmaRateFrags;
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    bf16x8 fa[NA], fb[NA];
#pragma unroll
    for (int j = 0; j < NA; ++j) {
        fa[j] = as_bf16x8(operands[(t * 8u + 2u * j) % n_vec]);
        fb[j] = as_bf16x8(operands[(t * 8u + 2u * j + 1u) % n_vec]);
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < NA; ++j) {
            c0 = mfma_bf16(fa[j], fb[j], c0);
            c1 = mfma_bf16(fa[j], fb[(j + 1) % NA], c1);
            c2 = mfma_bf16(fa[(j + 1) % NA], fb[j], c2);
            c3 = mfma_bf16(fa[(j + 2) % NA], fb[(j + 3) % NA], c3);
        }
    }
    sink[t] = c0[0] + c1[1] + c2[2] + c3[3];
}

// Second measurement aid: synthetic instruction streams with the attention kernels' instruction mixes, all
// operands in registers and all zero (so that the power limit plays no part), one workgroup per CU with one, two
// or three wavefronts per SIMD.  They answer what a kernel with such a mix can reach on this part at best when
// every MFMA is followed by its share of the vector and LDS work (the "uniform" streams), and what it costs to
// issue the same work the way the compiler orders a tile (the MFMAs in clumps, the softmax between them).
// MFMAs per pass of the loop and wavefront: kStreamProbeMfmas.
enum StreamMix {
    kStreamMfmaOnly = 0,
    kStreamFwdUniform = 1,      // per MFMA: 2 fma, 2 exp2, 2 add, 1 cvt_pk, 3/4 ds_read_b128
    kStreamFwdClumped = 2,      // per 32-key half: 8 MFMAs, the vector work of 32 elements, 8 MFMAs
    kStreamDqUniform = 3,       // per MFMA: 4/3 (fma, exp2, mul), 2/3 (add, cvt_pk, ds_read_b128)
    kStreamDqClumped = 4,       // per 32-key half: 16 MFMAs, the vector work of 64 elements, 8 MFMAs
    kStreamDkdvUniform = 5,     // per MFMA: 2 mul, 1 exp2, 1 cvt_pk, 3/4 ds_read_b128
    kStreamMixes = 6
};
constexpr int kStreamProbeMfmas = 48;
constexpr int kStreamProbeLdsBytes = 96 * 1024;      // more than half a CU's LDS: one workgroup per CU

template <int MIX>
__global__ __launch_bounds__(768) void stream_probe_kernel(float *sink, int iters) {
    extern __shared__ __attribute__((aligned(16))) char probe_lds[];
    // a zero the compiler cannot see through: constants would be materialised again right in front of their
    // first use, i.e. in front of the first inline-assembly MFMA and without the wait states a vector write needs
    // before an MFMA reads it
    float zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] = zero;
    union { u32x4 u; bf16x8 v; } zf;
    zf.u = u32x4{__float_as_uint(zero), __float_as_uint(zero), __float_as_uint(zero), __float_as_uint(zero)};
    bf16x8 fa = zf.v, fb = zf.v;
    float r[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) r[i] = zero;
    const float c = zero;
    u32x4 q0 = {0u, 0u, 0u, 0u};
    const uint32_t lds = lds_addr(probe_lds) + (threadIdx.x & 255u) * 16u;
    if (threadIdx.x < 256) *reinterpret_cast<u32x4 *>(probe_lds + threadIdx.x * 16) = q0;
    __syncthreads();
#define GPTOSS_P_MFMA(j) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[(j) & 3]) : "v"(fa), "v"(fb))
#define GPTOSS_P_EXP(i) asm volatile("v_exp_f32 %0, %0" : "+v"(r[(i) % 12]))
#define GPTOSS_P_MUL(i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(r[(i) % 12]) : "v"(c))
#define GPTOSS_P_FMA(i) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(r[(i) % 12]) : "v"(c))
#define GPTOSS_P_ADD(i) asm volatile("v_add_f32 %0, %0, %1" : "+v"(r[(i) % 12]) : "v"(c))
#define GPTOSS_P_CVT(i) asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1" : "+v"(r[(i) % 12]) : "v"(c))
#define GPTOSS_P_LDS() asm volatile("ds_read_b128 %0, %1" : "=v"(q0) : "v"(lds))
    // (the MFMAs below are inline assembly, so the compiler does not put the wait states between the vector
    // writes of their operands and their first read; taking the operands here, with the wait states, does)
    asm volatile("s_nop 7" : "+v"(fa), "+v"(fb), "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]));
    for (int it = 0; it < iters; ++it) {
        if constexpr (MIX == kStreamMfmaOnly || MIX == kStreamFwdUniform || MIX == kStreamDqUniform || MIX == kStreamDkdvUniform) {
#pragma unroll
            for (int j = 0; j < kStreamProbeMfmas; ++j) {
                GPTOSS_P_MFMA(j);
                if (MIX == kStreamFwdUniform) {
                    GPTOSS_P_FMA(j); GPTOSS_P_EXP(j); GPTOSS_P_ADD(j + 1); GPTOSS_P_FMA(j + 2); GPTOSS_P_EXP(j + 2); GPTOSS_P_ADD(j + 3); GPTOSS_P_CVT(j + 4);
                    if (j % 4 != 3) GPTOSS_P_LDS();
                }
                if (MIX == kStreamDqUniform) {
                    GPTOSS_P_FMA(j); GPTOSS_P_EXP(j); GPTOSS_P_MUL(j + 1);
                    if (j % 3 != 2) { GPTOSS_P_ADD(j + 3); GPTOSS_P_CVT(j + 2); GPTOSS_P_LDS(); }
                    if (j % 3 == 0) { GPTOSS_P_FMA(j + 4); GPTOSS_P_EXP(j + 4); GPTOSS_P_MUL(j + 5); }
                }
                if (MIX == kStreamDkdvUniform) {
                    GPTOSS_P_MUL(j); GPTOSS_P_EXP(j); GPTOSS_P_MUL(j + 1); GPTOSS_P_CVT(j + 2);
                    if (j % 4 != 3) GPTOSS_P_LDS();
                }
            }
        }
        if constexpr (MIX == kStreamFwdClumped) {
#pragma unroll
            for (int h = 0; h < 3; ++h) {
#pragma unroll
                for (int j = 0; j < 4; ++j) GPTOSS_P_LDS();
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_MFMA(j);
#pragma unroll
                for (int j = 0; j < 32; ++j) { GPTOSS_P_FMA(j); GPTOSS_P_EXP(j); GPTOSS_P_ADD(j + 1); if (j & 1) GPTOSS_P_CVT(j + 3); }
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_LDS();
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_MFMA(j);
            }
        }
        if constexpr (MIX == kStreamDqClumped) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_LDS();
#pragma unroll
                for (int j = 0; j < 16; ++j) GPTOSS_P_MFMA(j);
#pragma unroll
                for (int j = 0; j < 32; ++j) { GPTOSS_P_FMA(j); GPTOSS_P_EXP(j); GPTOSS_P_MUL(j + 1); if (j & 1) { GPTOSS_P_ADD(j + 2); GPTOSS_P_CVT(j + 3); } }
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_LDS();
#pragma unroll
                for (int j = 0; j < 8; ++j) GPTOSS_P_MFMA(j);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)");
    }
    // (the compiler does not know that the statements above are MFMAs: without these wait states the sums below
    // would read accumulators the last MFMAs have not written yet)
    asm volatile("s_nop 15\n\ts_nop 15");
#undef GPTOSS_P_MFMA
#undef GPTOSS_P_EXP
#undef GPTOSS_P_MUL
#undef GPTOSS_P_FMA
#undef GPTOSS_P_ADD
#undef GPTOSS_P_CVT
#undef GPTOSS_P_LDS
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) s += acc[j][0];
#pragma unroll
    for (int i = 0; i < 12; ++i) s += r[i];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s + __uint_as_float(q0[0]);
}

}  // namespace gptoss
