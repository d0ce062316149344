// Matrix-pipe ceiling probe for gfx950 (MI355X): a loop of nothing but the GEMM kernels' MFMA, in the GEMM's
// register pattern, with every operand held in registers: no LDS, no memory.  One workgroup of four wavefronts
// per compute unit (one per SIMD), like the 256x256 GEMM tile.  Two forms: v_mfma_f32_32x32x16_bf16 (a wavefront
// owns a 4 x 4 grid of 32x32 accumulators and multiplies four A fragments with four B fragments per k16 step) and
// v_mfma_f32_16x16x32_bf16 (8 x 8 accumulators of 16x16, eight fragments of each operand per k32 step).
//
// The operands of consecutive k16 steps rotate over SETS register-resident fragment sets filled
// with a pattern: zeros, one constant, or N(0, 0.02)-like pseudo-random bf16 values.  The rate
// the loop sustains with random operands is what the matrix pipes deliver under the board's power
// limit when the data toggles; with constant operands it is the limit of the pipes themselves.
#include "common.h"

namespace syn {

typedef unsigned int u32x4_probe_t __attribute__((ext_vector_type(4)));

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

// the same on 16x16x32 MFMAs: 128 per round, the flop of 64 of the larger ones.  The accumulators are named as AGPR
// tuples in inline assembly, as in the GEMM's K loop.
__global__ void __launch_bounds__(256) mfma16_rate_kernel(float* sink, int iters, int pattern) {
    typedef float f32x4_probe_t __attribute__((ext_vector_type(4)));
    f32x4_probe_t acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4_probe_t{0.f, 0.f, 0.f, 0.f};
    bf16x8_t fa[2][8], fb[2][8];
    const unsigned me = blockIdx.x * 256u + threadIdx.x;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            fa[s][i] = probe_fragment(pattern, (me * 2u + s) * 16u + i);
            fb[s][i] = probe_fragment(pattern, (me * 2u + s) * 16u + 8u + i);
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[s][j]), "v"(fa[s][i]));
    }
    // the compiler adds no wait states behind assembly MFMAs: a matrix op of N passes needs N + 3 of them (at
    // most 19) before a vector instruction may read its result
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) total += acc[i][j][0] + acc[i][j][3];
    sink[me] = total;
}

// HBM read ceiling probe: `STREAMS` read streams `stride_vecs` 16-byte groups apart, walked in the chunked
// reduce's access pattern - 256 lanes, four groups per lane and pass, every load of a pass issued
// before the first is used, non-temporal - with an exclusive-or in place of the adds and no result
// stream.  What it sustains is what the memory system gives that pattern of reads.
constexpr int kStreamThreads = 256;
constexpr int kStreamVecs = 4;

template <int STREAMS>
__global__ void __launch_bounds__(kStreamThreads)
read_streams_kernel(const u32x4_probe_t* __restrict__ base, int64_t stride_vecs, int64_t stream_vecs,
                    u32x4_probe_t* __restrict__ sink) {
    constexpr int64_t kGroup = (int64_t)kStreamThreads * kStreamVecs;
    u32x4_probe_t mix = {0u, 0u, 0u, 0u};
    for (int64_t g0 = (int64_t)blockIdx.x * kGroup; g0 + kGroup <= stream_vecs; g0 += (int64_t)gridDim.x * kGroup) {
        u32x4_probe_t parts[kStreamVecs][STREAMS];
#pragma unroll
        for (int u = 0; u < kStreamVecs; ++u)
#pragma unroll
            for (int i = 0; i < STREAMS; ++i)
                parts[u][i] = __builtin_nontemporal_load(base + (int64_t)i * stride_vecs + g0 + threadIdx.x + u * kStreamThreads);
#pragma unroll
        for (int u = 0; u < kStreamVecs; ++u)
#pragma unroll
            for (int i = 0; i < STREAMS; ++i) mix ^= parts[u][i];
    }
    // keeps the loads alive; a lane whose words happen to cancel leaves its note in the sink
    if ((mix.x ^ mix.y ^ mix.z ^ mix.w) == 0x9e3779b9u) sink[blockIdx.x] = mix;
}

}  // namespace syn

extern "C" int syn_probe_read_streams(const void* base, int64_t stream_bytes, int64_t stride_bytes, int32_t streams,
                                      int32_t workgroups, void* sink, syn_stream_t stream) {
    using namespace syn;
    if (base == nullptr || sink == nullptr || workgroups <= 0) return SYN_EINVAL;
    if (stream_bytes <= 0 || stream_bytes % (16 * kStreamThreads * kStreamVecs)) return SYN_EINVAL;
    if (streams != 1 && streams != 8) return SYN_EINVAL;
    if (stride_bytes < 0 || stride_bytes % 16 || !aligned16(base) || !aligned16(sink)) return SYN_EALIGN;
    const u32x4_probe_t* b = reinterpret_cast<const u32x4_probe_t*>(base);
    u32x4_probe_t* k = reinterpret_cast<u32x4_probe_t*>(sink);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (streams == 1)
        hipLaunchKernelGGL(read_streams_kernel<1>, dim3(workgroups), dim3(kStreamThreads), 0, s, b, stride_bytes / 16,
                           stream_bytes / 16, k);
    else
        hipLaunchKernelGGL(read_streams_kernel<8>, dim3(workgroups), dim3(kStreamThreads), 0, s, b, stride_bytes / 16,
                           stream_bytes / 16, k);
    return (int)hipGetLastError();
}

extern "C" int syn_probe_mfma_rate(float* sink, int32_t workgroups, int32_t iters, int32_t pattern,
                                   syn_stream_t stream) {
    using namespace syn;
    if (sink == nullptr || workgroups <= 0 || iters <= 0 || pattern < 0 || (pattern & 3) > 2 || pattern > 6) return SYN_EINVAL;
    if (pattern & 4)
        hipLaunchKernelGGL(mfma16_rate_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                           sink, iters, pattern & 3);
    else
        hipLaunchKernelGGL(mfma_rate_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), sink,
                           iters, pattern);
    return (int)hipGetLastError();
}
