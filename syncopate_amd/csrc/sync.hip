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

// Chunk copy that raises the chunk's flag itself: one kernel per chunk instead of a copy, a
// kernel boundary and a flag kernel.  Each workgroup copies its share with streaming stores and
// then takes a ticket with release semantics (its stores are written back and visible
// device-wide before the ticket moves); the workgroup that takes the last ticket sets the flag
// and puts the ticket counter back to zero for the next copy on the stream.  Write-through stores
// and a relaxed ticket (no write-back of the L2, which the compute kernel keeps dirty) were tried
// first: 8-byte write-through stores made the copy 1.5 times slower beside a running GEMM.
constexpr int kCopyFlagThreads = 1024;

__global__ void __launch_bounds__(kCopyFlagThreads)
copy_then_flag_kernel(uint64_t* __restrict__ dst, const u32x4_t* __restrict__ src, int64_t vecs,
                      uint32_t* ticket, uint64_t* flag, uint64_t value) {
    const int64_t stride = (int64_t)gridDim.x * kCopyFlagThreads;
    for (int64_t i = (int64_t)blockIdx.x * kCopyFlagThreads + threadIdx.x; i < vecs; i += 4 * stride) {
        u32x4_t v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (i + k * stride < vecs) v[k] = __builtin_nontemporal_load(src + i + k * stride);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (i + k * stride < vecs) {
                __builtin_nontemporal_store(v[k], reinterpret_cast<u32x4_t*>(dst) + i + k * stride);
            }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t taken = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        if (taken == gridDim.x - 1) {
            __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(flag, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

// A whole list of chunk copies, each followed by its flag, as ONE kernel: the workgroups walk the list
// in order, copy their share of a chunk with stores that go through the L2 to memory, wait for the
// stores' acknowledgements and take a ticket; the workgroup that takes a chunk's last ticket raises
// the chunk's flag.  Seven chunks then cost one kernel instead of fourteen - and, more to the point,
// no kernel boundary while the consumer runs: every kernel that starts or ends on the device brings
// an invalidate or a write-back of the L2s the consumer's panels live in.
struct CopyFlagOp {
    u32x4_t* dst;
    const u32x4_t* src;
    int64_t vecs;
    uint64_t* flag;
    uint64_t value;
    int64_t delay_ticks;        // wall-clock ticks to let pass before the chunk is copied (a slow link)
};

__device__ __forceinline__ void store16_through(u32x4_t* dst, u32x4_t v) {
    // a store of more than 8 bytes reads its data registers for two more issue slots (hence the s_nop)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
}

__global__ void __launch_bounds__(kCopyFlagThreads)
copy_flag_list_kernel(const CopyFlagOp* __restrict__ ops, int count, uint32_t* tickets) {
    const int64_t stride = (int64_t)gridDim.x * kCopyFlagThreads;
    CopyFlagOp next = ops[0];
    for (int k = 0; k < count; ++k) {
        const CopyFlagOp op = next;
        if (k + 1 < count) next = ops[k + 1];       // asked for now, needed a record later: short records are not a trip to memory each
        if (op.delay_ticks > 0) {
            const uint64_t t0 = wall_clock64();
            while ((int64_t)(wall_clock64() - t0) < op.delay_ticks) __builtin_amdgcn_s_sleep(32);
        }
        for (int64_t i = (int64_t)blockIdx.x * kCopyFlagThreads + threadIdx.x; i < op.vecs; i += 4 * stride) {
            u32x4_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i + u * stride < op.vecs) v[u] = __builtin_nontemporal_load(op.src + i + u * stride);
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i + u * stride < op.vecs) store16_through(op.dst + i + u * stride, v[u]);
        }
        // a record without a flag is a piece of a transfer whose last record carries it: a workgroup's stores
        // go out in record order, so the wait in front of that record's ticket covers them
        if (op.flag == nullptr) continue;
        __builtin_amdgcn_s_waitcnt(0x0070);          // vmcnt(0): this lane's stores have reached memory
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t taken = __hip_atomic_fetch_add(tickets + k, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (taken == gridDim.x - 1) {
                __hip_atomic_store(tickets + k, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(op.flag, op.value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
    }
}

// Box copy: a box of up to 5 dimensions, contiguous along the last one in source and
// destination, byte strides otherwise arbitrary; optionally dst += src by atomic adds, so that
// several senders may accumulate into one destination at a time.  The box is a list of rows
// (the last dimension); a row is cut into units of 16, 8, 4, 2 or 1 bytes - the largest that
// divides the row length, both base addresses and every stride - and the units are dealt to the
// lanes grid-stride, four in flight per lane.  Counterpart of the reference's SM-driven copies
// (comm_runtime/non_tma_persistent_copy.py:106-304, tma_persistent_copy.py), which the generated
// op lists use with copy_engine=False (SMCopyOp) and for reduce-scatter by direct reduction.
struct BoxParams {
    unsigned char* dst;
    const unsigned char* src;
    int64_t outer[4];          // extents of the dimensions in front of the last, leading ones padded with 1
    int64_t src_stride[4];     // in bytes
    int64_t dst_stride[4];
    int64_t row_units;         // units per row
    int64_t total_units;
    int32_t n_outer;           // how many of outer[] (counted from the back) are real
};

constexpr int kBoxThreads = 1024;
// loads in flight per lane: 64 bytes' worth, at most 16 (twice that gains nothing: a compute unit moves about
// 32 bytes per clock through its vector memory path either way)
template <int UNIT> struct BoxDepth { static constexpr int value = UNIT >= 16 ? 4 : (UNIT == 8 ? 8 : 16); };

template <int BYTES> struct BoxUnit;
template <> struct BoxUnit<16> { typedef u32x4_t type; };
template <> struct BoxUnit<8> { typedef uint64_t type; };
template <> struct BoxUnit<4> { typedef uint32_t type; };
template <> struct BoxUnit<2> { typedef uint16_t type; };
template <> struct BoxUnit<1> { typedef uint8_t type; };

// unit index -> byte offsets of the unit in source and destination
template <typename IdxT, int UNIT>
__device__ __forceinline__ void box_locate(const BoxParams& p, IdxT u, int64_t& so, int64_t& dof) {
    IdxT row = u / (IdxT)p.row_units;
    const IdxT col = u - row * (IdxT)p.row_units;
    so = (int64_t)col * UNIT;
    dof = so;
    for (int d = 3; d >= 4 - p.n_outer; --d) {
        const IdxT q = row / (IdxT)p.outer[d];
        const IdxT i = row - q * (IdxT)p.outer[d];
        so += (int64_t)i * p.src_stride[d];
        dof += (int64_t)i * p.dst_stride[d];
        row = q;
    }
}

template <typename IdxT, int UNIT>
__global__ void __launch_bounds__(kBoxThreads) box_copy_kernel(const BoxParams p) {
    typedef typename BoxUnit<UNIT>::type unit_t;
    constexpr int kBoxInFlight = BoxDepth<UNIT>::value;
    const IdxT total = (IdxT)p.total_units;
    const IdxT stride = (IdxT)gridDim.x * kBoxThreads;
    for (IdxT base = (IdxT)blockIdx.x * kBoxThreads + threadIdx.x; base < total; base += kBoxInFlight * stride) {
        unit_t v[kBoxInFlight];
        int64_t dof[kBoxInFlight];
#pragma unroll
        for (int k = 0; k < kBoxInFlight; ++k) {
            const IdxT u = base + (IdxT)k * stride;
            if (u < total) {
                int64_t so;
                box_locate<IdxT, UNIT>(p, u, so, dof[k]);
                v[k] = __builtin_nontemporal_load(reinterpret_cast<const unit_t*>(p.src + so));
            } else {
                dof[k] = -1;
            }
        }
#pragma unroll
        for (int k = 0; k < kBoxInFlight; ++k)
            if (dof[k] >= 0) *reinterpret_cast<unit_t*>(p.dst + dof[k]) = v[k];
    }
}

// dst += v for one unit of UNIT bytes holding elements of type T, by no-return atomics
template <typename T, int UNIT> struct BoxAdd;

template <int UNIT> struct BoxAdd<float, UNIT> {
    typedef typename BoxUnit<UNIT>::type unit_t;
    static __device__ __forceinline__ void apply(unsigned char* dst, unit_t v) {
        float vals[UNIT / 4];
        __builtin_memcpy(vals, &v, UNIT);
#pragma unroll
        for (int e = 0; e < UNIT / 4; ++e)
            __hip_atomic_fetch_add(reinterpret_cast<float*>(dst) + e, vals[e], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    }
};

template <typename T> __device__ __forceinline__ void packed_add(unsigned char* dst, uint32_t two);
template <> __device__ __forceinline__ void packed_add<__bf16>(unsigned char* dst, uint32_t two) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2* gptr;
    __builtin_amdgcn_global_atomic_fadd_v2bf16((gptr)dst, __builtin_bit_cast(v2, two));
}
template <> __device__ __forceinline__ void packed_add<_Float16>(unsigned char* dst, uint32_t two) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2* gptr;
    __builtin_amdgcn_global_atomic_fadd_v2f16((gptr)dst, __builtin_bit_cast(v2, two));
}

// 16-bit elements: pairs go through the packed atomics; a single element (a box that starts or
// ends on an odd element) through compare-and-swap on the 32-bit word around it
template <typename T, int UNIT> struct BoxAdd {
    typedef typename BoxUnit<UNIT>::type unit_t;
    static __device__ __forceinline__ void apply(unsigned char* dst, unit_t v) {
        if constexpr (UNIT >= 4) {
            uint32_t words[UNIT / 4];
            __builtin_memcpy(words, &v, UNIT);
#pragma unroll
            for (int e = 0; e < UNIT / 4; ++e) packed_add<T>(dst + 4 * e, words[e]);
        } else {
            const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
            uint32_t* word = reinterpret_cast<uint32_t*>(addr & ~(uintptr_t)3);
            const int shift = (addr & 2) ? 16 : 0;
            const float add = (float)__builtin_bit_cast(T, (uint16_t)v);
            uint32_t seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (;;) {
                const T cur = __builtin_bit_cast(T, (uint16_t)(seen >> shift));
                const uint32_t sum = __builtin_bit_cast(uint16_t, (T)((float)cur + add));
                const uint32_t want = (seen & ~(0xffffu << shift)) | (sum << shift);
                if (__hip_atomic_compare_exchange_strong(word, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT))
                    break;
            }
        }
    }
};

// dst += v for one unit by a plain read-modify-write: for a destination with one writer at a time
template <typename T, int UNIT>
__device__ __forceinline__ void box_add_plain(unsigned char* dst, typename BoxUnit<UNIT>::type v) {
    typedef typename BoxUnit<UNIT>::type unit_t;
    constexpr int kN = UNIT / (int)sizeof(T);
    unit_t cur = *reinterpret_cast<const unit_t*>(dst);
    T a[kN], b[kN];
    __builtin_memcpy(a, &cur, UNIT);
    __builtin_memcpy(b, &v, UNIT);
#pragma unroll
    for (int e = 0; e < kN; ++e) a[e] = (T)((float)a[e] + (float)b[e]);     // one rounding, as an add in T
    __builtin_memcpy(&cur, a, UNIT);
    *reinterpret_cast<unit_t*>(dst) = cur;
}

template <typename T, typename IdxT, int UNIT, bool ATOMIC>
__global__ void __launch_bounds__(kBoxThreads) box_add_kernel(const BoxParams p) {
    typedef typename BoxUnit<UNIT>::type unit_t;
    constexpr int kBoxInFlight = BoxDepth<UNIT>::value;
    const IdxT total = (IdxT)p.total_units;
    const IdxT stride = (IdxT)gridDim.x * kBoxThreads;
    for (IdxT base = (IdxT)blockIdx.x * kBoxThreads + threadIdx.x; base < total; base += kBoxInFlight * stride) {
        unit_t v[kBoxInFlight];
        int64_t dof[kBoxInFlight];
#pragma unroll
        for (int k = 0; k < kBoxInFlight; ++k) {
            const IdxT u = base + (IdxT)k * stride;
            if (u < total) {
                int64_t so;
                box_locate<IdxT, UNIT>(p, u, so, dof[k]);
                v[k] = __builtin_nontemporal_load(reinterpret_cast<const unit_t*>(p.src + so));
            } else {
                dof[k] = -1;
            }
        }
#pragma unroll
        for (int k = 0; k < kBoxInFlight; ++k) {
            if (dof[k] < 0) continue;
            if constexpr (ATOMIC) BoxAdd<T, UNIT>::apply(p.dst + dof[k], v[k]);
            else box_add_plain<T, UNIT>(p.dst + dof[k], v[k]);
        }
    }
}

template <typename IdxT>
static void launch_box_copy(const BoxParams& p, int unit, int blocks, hipStream_t s) {
    const dim3 g(blocks), b(kBoxThreads);
    switch (unit) {
        case 16: hipLaunchKernelGGL((box_copy_kernel<IdxT, 16>), g, b, 0, s, p); break;
        case 8: hipLaunchKernelGGL((box_copy_kernel<IdxT, 8>), g, b, 0, s, p); break;
        case 4: hipLaunchKernelGGL((box_copy_kernel<IdxT, 4>), g, b, 0, s, p); break;
        case 2: hipLaunchKernelGGL((box_copy_kernel<IdxT, 2>), g, b, 0, s, p); break;
        default: hipLaunchKernelGGL((box_copy_kernel<IdxT, 1>), g, b, 0, s, p); break;
    }
}

template <typename T, typename IdxT, bool ATOMIC>
static void launch_box_add(const BoxParams& p, int unit, int blocks, hipStream_t s) {
    const dim3 g(blocks), b(kBoxThreads);
    if (unit == 16) {
        if constexpr (!ATOMIC) hipLaunchKernelGGL((box_add_kernel<T, IdxT, 16, false>), g, b, 0, s, p);
    } else if (unit == 8) {
        if constexpr (!ATOMIC) hipLaunchKernelGGL((box_add_kernel<T, IdxT, 8, false>), g, b, 0, s, p);
    } else if (unit == 4) {
        hipLaunchKernelGGL((box_add_kernel<T, IdxT, 4, ATOMIC>), g, b, 0, s, p);
    } else {
        if constexpr (sizeof(T) == 2) hipLaunchKernelGGL((box_add_kernel<T, IdxT, 2, ATOMIC>), g, b, 0, s, p);
    }
}

template <typename T>
static void launch_box_add_any(const BoxParams& p, int unit, int blocks, bool narrow, bool atomic, hipStream_t s) {
    if (atomic) {
        if (narrow) launch_box_add<T, uint32_t, true>(p, unit, blocks, s);
        else launch_box_add<T, uint64_t, true>(p, unit, blocks, s);
    } else {
        if (narrow) launch_box_add<T, uint32_t, false>(p, unit, blocks, s);
        else launch_box_add<T, uint64_t, false>(p, unit, blocks, s);
    }
}

// Where did each workgroup run?  out[2 b] = the hardware id word of workgroup b's first
// wavefront (compute unit, shader array and shader engine in bits 8..15), out[2 b + 1] = the id
// of its XCD.  The workgroups stay for `dwell` short sleeps so that a grid spreads over every
// compute unit its stream may use.
__global__ void __launch_bounds__(256) where_kernel(uint32_t* out, int dwell) {
    uint32_t hw, xcd;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcd));
    for (int i = 0; i < dwell; ++i) __builtin_amdgcn_s_sleep(16);
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = hw;
        out[2 * blockIdx.x + 1] = xcd;
    }
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

int syn_copy_flag_async(void* dst, const void* src, int64_t nbytes, uint64_t* flag, uint64_t value,
                        uint32_t* ticket, int32_t num_blocks, syn_stream_t stream) {
    if (nbytes <= 0 || !dst || !src || !flag || !ticket) return SYN_EINVAL;
    if (num_blocks <= 0 || num_blocks > 4096) return SYN_EINVAL;
    if (nbytes % 16 || !syn::aligned16(dst) || !syn::aligned16(src)) return SYN_EALIGN;
    const int64_t vecs = nbytes / 16;
    const int64_t needed = (vecs + syn::kCopyFlagThreads - 1) / syn::kCopyFlagThreads;
    const int blocks = (int)(needed < num_blocks ? needed : num_blocks);
    hipLaunchKernelGGL(syn::copy_then_flag_kernel, dim3(blocks), dim3(syn::kCopyFlagThreads), 0,
                       reinterpret_cast<hipStream_t>(stream), reinterpret_cast<uint64_t*>(dst),
                       reinterpret_cast<const syn::u32x4_t*>(src), vecs, ticket, flag, value);
    return (int)hipGetLastError();
}

int syn_copy_flag_list_async(const syn_copy_flag_op* ops, int32_t count, uint32_t* tickets, int32_t num_blocks,
                             syn_stream_t stream) {
    static_assert(sizeof(syn_copy_flag_op) == sizeof(syn::CopyFlagOp), "the kernel's record is the header's");
    if (!ops || !tickets || count <= 0 || count > 4096) return SYN_EINVAL;
    if (num_blocks <= 0 || num_blocks > 4096) return SYN_EINVAL;
    hipLaunchKernelGGL(syn::copy_flag_list_kernel, dim3(num_blocks), dim3(syn::kCopyFlagThreads), 0,
                       reinterpret_cast<hipStream_t>(stream), reinterpret_cast<const syn::CopyFlagOp*>(ops), count,
                       tickets);
    return (int)hipGetLastError();
}

int syn_box_copy_async(void* dst, const void* src, int32_t ndim, const int64_t* shape,
                       const int64_t* src_strides, const int64_t* dst_strides, int32_t elem_kind,
                       int32_t reduce_mode, int32_t num_blocks, syn_stream_t stream) {
    using namespace syn;
    if (!dst || !src || !shape || !src_strides || !dst_strides) return SYN_EINVAL;
    if (ndim < 1 || ndim > 5) return SYN_EINVAL;
    if (num_blocks <= 0) return SYN_EINVAL;
    int elem = 0;
    switch (elem_kind) {
        case SYN_ELEM_BF16: case SYN_ELEM_FP16: case SYN_ELEM_2B: elem = 2; break;
        case SYN_ELEM_FP32: case SYN_ELEM_4B: elem = 4; break;
        case SYN_ELEM_1B: elem = 1; break;
        case SYN_ELEM_8B: elem = 8; break;
        default: return SYN_EINVAL;
    }
    if (reduce_mode < SYN_BOX_COPY || reduce_mode > SYN_BOX_ADD_EXCLUSIVE) return SYN_EINVAL;
    const bool sum = reduce_mode != SYN_BOX_COPY;
    const bool atomic = reduce_mode == SYN_BOX_ADD_ATOMIC;
    if (sum && elem_kind != SYN_ELEM_BF16 && elem_kind != SYN_ELEM_FP16 && elem_kind != SYN_ELEM_FP32)
        return SYN_EINVAL;                                   // sums need a float type
    if (src_strides[ndim - 1] != 1 || dst_strides[ndim - 1] != 1) return SYN_EINVAL;   // rows are contiguous
    if (shape[ndim - 1] <= 0) return SYN_EINVAL;
    const uintptr_t da = reinterpret_cast<uintptr_t>(dst), sa = reinterpret_cast<uintptr_t>(src);
    if (da % elem || sa % elem) return SYN_EINVAL;
    BoxParams p;
    p.dst = reinterpret_cast<unsigned char*>(dst);
    p.src = reinterpret_cast<const unsigned char*>(src);
    p.n_outer = ndim - 1;
    const int64_t row_bytes = shape[ndim - 1] * elem;
    // every address of the box is a multiple of the unit when these all are
    uint64_t mix = (uint64_t)da | (uint64_t)sa | (uint64_t)row_bytes | 16u;
    int64_t rows = 1;
    for (int d = 0; d < 4; ++d) {
        const int from = ndim - 1 - (4 - d);     // outer[3] is the dimension next to the last
        if (from >= 0) {
            if (shape[from] <= 0 || src_strides[from] < 0 || dst_strides[from] < 0) return SYN_EINVAL;
            p.outer[d] = shape[from];
            p.src_stride[d] = src_strides[from] * elem;
            p.dst_stride[d] = dst_strides[from] * elem;
            if (shape[from] > 1) mix |= (uint64_t)p.src_stride[d] | (uint64_t)p.dst_stride[d];
            rows *= shape[from];
        } else {
            p.outer[d] = 1;
            p.src_stride[d] = p.dst_stride[d] = 0;
        }
    }
    int unit = (int)(mix & (~mix + 1));          // lowest set bit: 1, 2, 4, 8 or 16
    // atomic sums go by 4-byte words (a pair of 16-bit elements, one float): the lanes of a
    // wavefront then hit consecutive words, which the atomic units take 3.6 times faster than
    // four words per lane (measured on a 134 MB box); a single 16-bit element where the box
    // starts or ends on an odd one
    if (atomic && unit > 4) unit = 4;
    p.row_units = row_bytes / unit;
    p.total_units = rows * p.row_units;
    const int64_t needed = (p.total_units + kBoxThreads - 1) / kBoxThreads;
    const int blocks = (int)(needed < num_blocks ? needed : num_blocks);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    // 32-bit index arithmetic is several times cheaper; below 2^27 units no index of the
    // grid-stride loop (up to 16 deep, stride <= total + 1023) can wrap
    const bool narrow = p.total_units < (int64_t)1 << 27;
    if (!sum) {
        if (narrow) launch_box_copy<uint32_t>(p, unit, blocks, s);
        else launch_box_copy<uint64_t>(p, unit, blocks, s);
    } else if (elem_kind == SYN_ELEM_BF16) {
        launch_box_add_any<__bf16>(p, unit, blocks, narrow, atomic, s);
    } else if (elem_kind == SYN_ELEM_FP16) {
        launch_box_add_any<_Float16>(p, unit, blocks, narrow, atomic, s);
    } else {
        launch_box_add_any<float>(p, unit, blocks, narrow, atomic, s);
    }
    return (int)hipGetLastError();
}

int syn_flag_set(uint64_t* flag, uint64_t value, syn_stream_t stream) {
    if (!flag) return SYN_EINVAL;
    hipLaunchKernelGGL(syn::flag_set_kernel, dim3(1), dim3(64), 0,
                       reinterpret_cast<hipStream_t>(stream), flag, value);
    return (int)hipGetLastError();
}

int syn_flag_write_value(uint64_t* flag, uint64_t value, syn_stream_t stream) {
    if (!flag) return SYN_EINVAL;
    return (int)hipStreamWriteValue64(reinterpret_cast<hipStream_t>(stream), flag, value, 0);
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

int syn_stream_create_cu_mask(const uint32_t* mask, uint32_t words, syn_stream_t* stream) {
    if (!mask || !stream || words == 0 || words > 32) return SYN_EINVAL;
    uint32_t any = 0;
    for (uint32_t i = 0; i < words; ++i) any |= mask[i];
    if (!any) return SYN_EINVAL;                       // a stream without compute units never runs a kernel
    hipStream_t s = nullptr;
    const hipError_t err = hipExtStreamCreateWithCUMask(&s, words, mask);
    if (err != hipSuccess) return (int)err;
    *stream = reinterpret_cast<syn_stream_t>(s);
    return 0;
}

int syn_stream_destroy(syn_stream_t stream) {
    if (!stream) return SYN_EINVAL;
    return (int)hipStreamDestroy(reinterpret_cast<hipStream_t>(stream));
}

int syn_where_async(uint32_t* out, int32_t workgroups, int32_t dwell, syn_stream_t stream) {
    if (!out || workgroups <= 0 || workgroups > 65536 || dwell < 0 || dwell > 4096) return SYN_EINVAL;
    hipLaunchKernelGGL(syn::where_kernel, dim3(workgroups), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), out, dwell);
    return (int)hipGetLastError();
}

int syn_version(void) { return 100; }

}  // extern "C"
