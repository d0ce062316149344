// Matrix-pipe ceiling probe for gfx950 (MI355X): a loop of nothing but the GEMM kernels' MFMA
// (v_mfma_f32_32x32x16_bf16), in the GEMM's register pattern - a wavefront owns a 4 x 4 grid of
// 32x32 accumulators and multiplies four A fragments with four B fragments per k16 step - with
// every operand held in registers: no LDS, no memory.  One workgroup of four wavefronts per
// compute unit (one per SIMD), like the 256x256 GEMM tile.
//
// The operands of consecutive k16 steps rotate over SETS register-resident fragment sets filled
// with a pattern: zeros, one constant, or N(0, 0.02)-like pseudo-random bf16 values.  The rate
// the loop sustains with random operands is what the matrix pipes deliver under the board's power
// limit when the data toggles; with constant operands it is the limit of the pipes themselves.
#include "common.h"

namespace syn {

constexpr int kProbeSets = 4;

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

// pattern 0: zeros; 1: every element 1.0; 2: pseudo-random, roughly N(0, 0.02) (sum of four uniforms)
__device__ __forceinline__ bf16x8_t probe_fragment(int pattern, unsigned seed) {
    bf16x8_t f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float v = 0.f;
        if (pattern == 1) v = 1.0f;
        if (pattern == 2) {
            const unsigned h = probe_hash(seed * 8u + e);
            const float u = (float)(h & 0xff) + (float)((h >> 8) & 0xff) + (float)((h >> 16) & 0xff) + (float)(h >> 24);
            v = (u - 510.f) * (0.02f / 147.8f);      // variance of the sum of four U{0..255}: 4 * 5461.25
        }
        f[e] = (__bf16)v;
    }
    return f;
}

__global__ void __launch_bounds__(256) mfma_rate_kernel(float* sink, int iters, int pattern) {
    f32x16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    bf16x8_t fa[kProbeSets][4], fb[kProbeSets][4];
    const unsigned me = blockIdx.x * 256u + threadIdx.x;
#pragma unroll
    for (int s = 0; s < kProbeSets; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            fa[s][i] = probe_fragment(pattern, (me * kProbeSets + s) * 8u + i);
            fb[s][i] = probe_fragment(pattern, (me * kProbeSets + s) * 8u + 4u + i);
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < kProbeSets; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[s][j], fa[s][i], acc[i][j], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total += acc[i][j][0] + acc[i][j][7];
    sink[me] = total;
}

}  // namespace syn

extern "C" int syn_probe_mfma_rate(float* sink, int32_t workgroups, int32_t iters, int32_t pattern,
                                   syn_stream_t stream) {
    using namespace syn;
    if (sink == nullptr || workgroups <= 0 || iters <= 0 || pattern < 0 || pattern > 2) return SYN_EINVAL;
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), sink,
                       iters, pattern);
    return (int)hipGetLastError();
}
