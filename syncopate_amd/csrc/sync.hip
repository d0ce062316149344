// Stream-side primitives of the single-GPU producer: the counterparts of the
// reference runtime's cudaMemcpyAsync, cuStreamWriteValue and cuStreamWaitValue
// (syncopate/communication/comm_runtime/communication_context.py:129-160),
// written as one-wavefront kernels so they order with the copies on a stream.
#include "common.h"

namespace syn {

// The flag follows a copy on the same stream, and a kernel (or copy) that has completed has
// already written its data back: the flag itself only has to go through to memory.  A release
// fence here would write back the whole L2 of this XCD, dirty with whatever the compute kernel
// is storing at the time - microseconds per flag.
__global__ void __launch_bounds__(64) flag_set_kernel(uint64_t* flag, uint64_t value) {
    if (threadIdx.x == 0)
        __hip_atomic_store(flag, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ void __launch_bounds__(64)
flag_wait_kernel(const uint64_t* flag, uint64_t value, int64_t budget_ticks, int32_t* status) {
    if (threadIdx.x == 0) {
        if (!spin_until_equal(flag, value, budget_ticks))
            report_status(status, SYN_STATUS_SPIN_TIMEOUT, -1, -1, -1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// Chunk copy on compute units with streaming (non-temporal) accesses: the chunk passes
// through without displacing the consumer's working set from L2.  Small footprint (256
// threads, a handful of registers, no LDS) so that a workgroup fits beside resident
// compute workgroups.
__global__ void __launch_bounds__(256)
stream_copy_kernel(u32x4_t* __restrict__ dst, const u32x4_t* __restrict__ src, int64_t vecs) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < vecs; i += 4 * stride) {
        const u32x4_t a = __builtin_nontemporal_load(src + i);
        const u32x4_t b = __builtin_nontemporal_load(src + i + stride);
        const u32x4_t c = __builtin_nontemporal_load(src + i + 2 * stride);
        const u32x4_t d = __builtin_nontemporal_load(src + i + 3 * stride);
        __builtin_nontemporal_store(a, dst + i);
        __builtin_nontemporal_store(b, dst + i + stride);
        __builtin_nontemporal_store(c, dst + i + 2 * stride);
        __builtin_nontemporal_store(d, dst + i + 3 * stride);
    }
    for (; i < vecs; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

__global__ void __launch_bounds__(64) delay_kernel(int64_t ticks) {
    if (threadIdx.x == 0) {
        const uint64_t t0 = wall_clock64();
        while ((int64_t)(wall_clock64() - t0) < ticks) __builtin_amdgcn_s_sleep(16);
    }
}

}  // namespace syn

extern "C" {

int syn_copy_async(void* dst, const void* src, int64_t nbytes, syn_stream_t stream) {
    if (nbytes < 0 || (nbytes > 0 && (!dst || !src))) return SYN_EINVAL;
    if (nbytes == 0) return 0;
    return (int)hipMemcpyAsync(dst, src, (size_t)nbytes, hipMemcpyDeviceToDevice,
                               reinterpret_cast<hipStream_t>(stream));
}

int syn_copy_kernel_async(void* dst, const void* src, int64_t nbytes, int32_t num_blocks,
                          syn_stream_t stream) {
    if (nbytes < 0 || (nbytes > 0 && (!dst || !src))) return SYN_EINVAL;
    if (num_blocks <= 0 || num_blocks > 4096) return SYN_EINVAL;
    if (nbytes % 16 || !syn::aligned16(dst) || !syn::aligned16(src)) return SYN_EALIGN;
    if (nbytes == 0) return 0;
    hipLaunchKernelGGL(syn::stream_copy_kernel, dim3(num_blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), reinterpret_cast<syn::u32x4_t*>(dst),
                       reinterpret_cast<const syn::u32x4_t*>(src), nbytes / 16);
    return (int)hipGetLastError();
}

int syn_flag_set(uint64_t* flag, uint64_t value, syn_stream_t stream) {
    if (!flag) return SYN_EINVAL;
    hipLaunchKernelGGL(syn::flag_set_kernel, dim3(1), dim3(64), 0,
                       reinterpret_cast<hipStream_t>(stream), flag, value);
    return (int)hipGetLastError();
}

int syn_flag_wait(const uint64_t* flag, uint64_t value, int64_t spin_timeout_us, int32_t* status,
                  syn_stream_t stream) {
    if (!flag) return SYN_EINVAL;
    hipLaunchKernelGGL(syn::flag_wait_kernel, dim3(1), dim3(64), 0,
                       reinterpret_cast<hipStream_t>(stream), flag, value,
                       syn::timeout_ticks(spin_timeout_us), status);
    return (int)hipGetLastError();
}

int syn_delay_us(int64_t us, syn_stream_t stream) {
    if (us < 0 || us > 1000000) return SYN_EINVAL;   // a delay is a model of link time, not a sleep
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0)
        khz = 100000;
    hipLaunchKernelGGL(syn::delay_kernel, dim3(1), dim3(64), 0,
                       reinterpret_cast<hipStream_t>(stream), us * (int64_t)khz / 1000);
    return (int)hipGetLastError();
}

int syn_version(void) { return 100; }

}  // extern "C"
