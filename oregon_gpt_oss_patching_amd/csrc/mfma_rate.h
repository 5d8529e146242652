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

}  // namespace gptoss
