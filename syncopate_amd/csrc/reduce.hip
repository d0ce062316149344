// Chunked ring reduce of GEMM+RS for gfx950 (tests/test_gemm_rs.py:22-72 of the reference):
//   out[e] = local[rank*chunk + e] + sum_{i=1..W-1} recv[((rank+i) % W)*chunk + e]
// A pure HBM stream: W reads and one write of 16 bytes per lane and element group; the streams are walked
// skewed against each other (see skewed_walk), what is left over in passes of four groups per lane.
#include "common.h"

namespace syn {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kReduceThreads = 256;
constexpr int kMaxWorld = 16;

template <typename T>
__device__ __forceinline__ float to_f32(T x) { return (float)x; }

// the running sum of one 16-byte group: eight fp32 values, added to in ring order
template <typename T>
__device__ __forceinline__ void sum_begin(float (&acc)[8], const u32x4_t first) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    const vec8 v = __builtin_bit_cast(vec8, first);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = (float)v[e];
}

template <typename T, bool ROUND_EACH>
__device__ __forceinline__ void sum_add(float (&acc)[8], const u32x4_t part) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    const vec8 v = __builtin_bit_cast(vec8, part);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        float s = acc[e] + (float)v[e];
        // fp32 add followed by round-to-nearest-even equals a correctly
        // rounded add in the 16-bit type (both operands have <= 11 bits)
        if (ROUND_EACH) s = (float)(T)s;
        acc[e] = s;
    }
}

template <typename T>
__device__ __forceinline__ u32x4_t sum_end(const float (&acc)[8]) {
    typedef T vec8 __attribute__((ext_vector_type(8)));
    vec8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (T)acc[e];
    return __builtin_bit_cast(u32x4_t, r);
}

template <typename T, bool ROUND_EACH>
__device__ __forceinline__ u32x4_t add8(const u32x4_t* parts, int count) {
    float acc[8];
    sum_begin<T>(acc, parts[0]);
    for (int i = 1; i < count; ++i) sum_add<T, ROUND_EACH>(acc, parts[i]);
    return sum_end<T>(acc);
}

constexpr int kVecsPerThread = 4;      // 16-byte groups per lane and pass of the plain walk: 4 x W loads in flight
constexpr int kSkewBlocks = 8;         // blocks of 256 16-byte groups (4 KB per stream) a workgroup takes in one skewed walk

// The received blocks lie a whole number of MiB apart (the reference's [W, rows, N] layout), so element e of
// every stream sits in the same DRAM bank and channel, in another row: W reads of one element at one time are W
// row conflicts in one bank.  A workgroup therefore walks its 32 KB of every stream SKEWED: in step t it reads
// block t - i of stream i (4 KB further on for each earlier stream), adds it to that block's running sum -
// still own block first, then the received ones in ring order - and stores a block once its last stream is in.
// Read alone, the eight streams come at 6.6-6.7 TB/s this way against 6.1-6.2 at equal offsets: what the layout
// with 4 KiB between the blocks gives (syn_ring_reduce_strided), without asking the caller for it.
template <typename T, bool ROUND_EACH, int W>
__device__ __forceinline__ void skewed_walk(const u32x4_t* __restrict__ recv, const u32x4_t* __restrict__ own,
                                            u32x4_t* __restrict__ out, int rank, int64_t recv_stride_vecs, int64_t v0) {
    float acc[kSkewBlocks][8];
    u32x4_t even[W], odd[W];
    auto stream = [&](int i) __attribute__((always_inline)) -> const u32x4_t* {
        if (i == 0) return own;
        int src = rank + i;
        if (src >= W) src -= W;
        return recv + (int64_t)src * recv_stride_vecs;
    };
    auto issue = [&](const int t, u32x4_t (&dst)[W]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const int b = t - i;
            if (b >= 0 && b < kSkewBlocks) dst[i] = __builtin_nontemporal_load(stream(i) + v0 + b * kReduceThreads);
        }
    };
    auto take = [&](const int t, const u32x4_t (&src)[W]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const int b = t - i;
            if (b >= 0 && b < kSkewBlocks) {
                if (i == 0) sum_begin<T>(acc[b], src[0]);
                else sum_add<T, ROUND_EACH>(acc[b], src[i]);
                if (i == W - 1) __builtin_nontemporal_store(sum_end<T>(acc[b]), out + v0 + b * kReduceThreads);
            }
        }
    };
    constexpr int kSteps = kSkewBlocks + W - 1;
    issue(0, even);
#pragma unroll
    for (int t = 0; t < kSteps; ++t) {
        // the next step's loads go out before this step's are used
        if (t + 1 < kSteps) {
            if (t & 1) issue(t + 1, even);
            else issue(t + 1, odd);
        }
        if (t & 1) take(t, odd);
        else take(t, even);
    }
}

template <typename T, bool ROUND_EACH, int W>
__global__ void __launch_bounds__(kReduceThreads)
ring_reduce_kernel(const u32x4_t* __restrict__ recv, const u32x4_t* __restrict__ local,
                   u32x4_t* __restrict__ out, int world, int rank, int64_t chunk_vecs, int64_t recv_stride_vecs, int skew) {
    // W > 0: world known at compile time (fully unrolled loads); W == 0: generic
    constexpr int kParts = W > 0 ? W : kMaxWorld;
    constexpr int64_t kGroup = (int64_t)kReduceThreads * kVecsPerThread;
    constexpr int64_t kSuper = (int64_t)kReduceThreads * kSkewBlocks;
    const int w = W > 0 ? W : world;
    const u32x4_t* own = local + (int64_t)rank * chunk_vecs;
    int64_t done = 0;                      // 16-byte groups covered by skewed walks
    if (W > 0 && skew) {
        done = chunk_vecs / kSuper * kSuper;
        for (int64_t s0 = (int64_t)blockIdx.x * kSuper; s0 < done; s0 += (int64_t)gridDim.x * kSuper)
            skewed_walk<T, ROUND_EACH, W == 0 ? 2 : W>(recv, own, out, rank, recv_stride_vecs, s0 + threadIdx.x);
    }
    for (int64_t g0 = done + (int64_t)blockIdx.x * kGroup; g0 < chunk_vecs; g0 += (int64_t)gridDim.x * kGroup) {
        const int64_t v0 = g0 + threadIdx.x;
        if (W > 0 && g0 + kGroup <= chunk_vecs) {
            // a full group (world known at compile time): every load of the pass is issued before the first add
            u32x4_t parts[kVecsPerThread][kParts];
#pragma unroll
            for (int u = 0; u < kVecsPerThread; ++u) {
                const int64_t v = v0 + u * kReduceThreads;
                parts[u][0] = __builtin_nontemporal_load(own + v);
#pragma unroll
                for (int i = 1; i < kParts; ++i) {
                    if (i < w) {
                        int src = rank + i;
                        if (src >= w) src -= w;
                        parts[u][i] = __builtin_nontemporal_load(recv + (int64_t)src * recv_stride_vecs + v);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kVecsPerThread; ++u)
                __builtin_nontemporal_store(add8<T, ROUND_EACH>(parts[u], w), out + v0 + u * kReduceThreads);
        } else if (W > 0) {
            for (int64_t v = v0; v < chunk_vecs; v += kReduceThreads) {
                u32x4_t parts[kParts];
                parts[0] = __builtin_nontemporal_load(own + v);
#pragma unroll
                for (int i = 1; i < kParts; ++i) {
                    int src = rank + i;
                    if (src >= w) src -= w;
                    parts[i] = __builtin_nontemporal_load(recv + (int64_t)src * recv_stride_vecs + v);
                }
                __builtin_nontemporal_store(add8<T, ROUND_EACH>(parts, w), out + v);
            }
        } else {
            // any world size: the received blocks four at a time (registers the compiler can name: an array of
            // `world` parts indexed by a run-time count would live in scratch memory), added in ring order
            for (int64_t v = v0; v < chunk_vecs && v < g0 + kGroup; v += kReduceThreads) {
                float acc[8];
                sum_begin<T>(acc, __builtin_nontemporal_load(own + v));
                for (int i = 1; i < w; i += 4) {
                    u32x4_t parts[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (i + j < w) {
                            int src = rank + i + j;
                            if (src >= w) src -= w;
                            parts[j] = __builtin_nontemporal_load(recv + (int64_t)src * recv_stride_vecs + v);
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (i + j < w) sum_add<T, ROUND_EACH>(acc, parts[j]);
                }
                __builtin_nontemporal_store(sum_end<T>(acc), out + v);
            }
        }
    }
}

template <typename T, bool ROUND_EACH>
static int launch_reduce(const void* recv, const void* local, void* out, int world, int rank,
                         int64_t chunk_vecs, int64_t recv_stride_vecs, hipStream_t stream) {
    // a workgroup takes 2048 16-byte groups per skewed walk (1024 per pass of the plain walk); two workgroups per
    // CU, beyond that they loop
    const int64_t group = (int64_t)kReduceThreads * kVecsPerThread;
    int64_t blocks = (chunk_vecs + group - 1) / group;
    const int64_t cap = 256 * 2;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    // skewed walks where they fill the grid (a chunk of at least 16 MiB per stream) and the received blocks lie a
    // multiple of 64 KiB apart; smaller chunks keep the plain walk, whose workgroups are twice as many, and so do
    // blocks that the caller has already moved out of each other's banks (the 4 KiB of padded_receive_buffer would
    // be undone by a skew of 4 KiB blocks)
    const int skew = (chunk_vecs / ((int64_t)kReduceThreads * kSkewBlocks) >= cap && recv_stride_vecs % 4096 == 0) ? 1 : 0;
    const dim3 grid((unsigned)blocks), block(kReduceThreads);
    const u32x4_t* r = reinterpret_cast<const u32x4_t*>(recv);
    const u32x4_t* l = reinterpret_cast<const u32x4_t*>(local);
    u32x4_t* o = reinterpret_cast<u32x4_t*>(out);
    switch (world) {
        case 2: hipLaunchKernelGGL((ring_reduce_kernel<T, ROUND_EACH, 2>), grid, block, 0, stream, r, l, o, world, rank, chunk_vecs, recv_stride_vecs, skew); break;
        case 4: hipLaunchKernelGGL((ring_reduce_kernel<T, ROUND_EACH, 4>), grid, block, 0, stream, r, l, o, world, rank, chunk_vecs, recv_stride_vecs, skew); break;
        case 8: hipLaunchKernelGGL((ring_reduce_kernel<T, ROUND_EACH, 8>), grid, block, 0, stream, r, l, o, world, rank, chunk_vecs, recv_stride_vecs, skew); break;
        default: hipLaunchKernelGGL((ring_reduce_kernel<T, ROUND_EACH, 0>), grid, block, 0, stream, r, l, o, world, rank, chunk_vecs, recv_stride_vecs, 0); break;
    }
    return (int)hipGetLastError();
}

}  // namespace syn

extern "C" int syn_ring_reduce_strided(const void* recv, int64_t recv_block_stride, const void* local, void* out,
                                       int32_t world, int32_t rank, int64_t rows_per_rank, int64_t N, int32_t dtype,
                                       int32_t acc_mode, syn_stream_t stream) {
    using namespace syn;
    if (!recv || !local || !out) return SYN_EINVAL;
    if (world < 1 || world > kMaxWorld || rank < 0 || rank >= world) return SYN_EINVAL;
    if (rows_per_rank <= 0 || N <= 0) return SYN_EINVAL;
    if (acc_mode != 0 && acc_mode != 1) return SYN_EINVAL;
    const int64_t elems = rows_per_rank * N;
    if (recv_block_stride < elems) return SYN_EINVAL;
    if (elems % 8 || recv_block_stride % 8) return SYN_EALIGN;
    if (!aligned16(recv) || !aligned16(local) || !aligned16(out)) return SYN_EALIGN;
    const int64_t vecs = elems / 8, stride = recv_block_stride / 8;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (dtype == SYN_DTYPE_BF16) {
        return acc_mode == 0 ? launch_reduce<__bf16, true>(recv, local, out, world, rank, vecs, stride, s)
                             : launch_reduce<__bf16, false>(recv, local, out, world, rank, vecs, stride, s);
    }
    if (dtype == SYN_DTYPE_FP16) {
        return acc_mode == 0 ? launch_reduce<_Float16, true>(recv, local, out, world, rank, vecs, stride, s)
                             : launch_reduce<_Float16, false>(recv, local, out, world, rank, vecs, stride, s);
    }
    return SYN_EINVAL;
}

extern "C" int syn_ring_reduce(const void* recv, const void* local, void* out, int32_t world,
                               int32_t rank, int64_t rows_per_rank, int64_t N, int32_t dtype,
                               int32_t acc_mode, syn_stream_t stream) {
    if (rows_per_rank <= 0 || N <= 0) return SYN_EINVAL;
    return syn_ring_reduce_strided(recv, rows_per_rank * N, local, out, world, rank, rows_per_rank, N, dtype, acc_mode,
                                   stream);
}
