// Shared device/host helpers for the gfx950 kernels of libsyncopate_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/syncopate_hip.h"

namespace syn {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kWaveSize = 64;
constexpr int kNumXcd = 8;                     // MI355X: 8 XCDs x 32 CUs, one L2 each
constexpr int64_t kDefaultSpinTimeoutUs = 2000000;

// wall_clock64() ticks at a fixed rate (100 MHz on gfx9); the host converts
// microseconds to ticks with the rate the device reports.
inline int64_t timeout_ticks(int64_t timeout_us) {
    if (timeout_us <= 0) timeout_us = kDefaultSpinTimeoutUs;
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess) return timeout_us * 100;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0)
        khz = 100000;
    return timeout_us * (int64_t)khz / 1000;
}

// Spin (one lane) until *flag == expect or the tick budget runs out.  The poll
// is a relaxed agent-scope load so that waiting does not keep invalidating
// caches; the caller issues the acquire fence once the flag has been seen.
// Returns true when the flag was observed.
__device__ __forceinline__ bool spin_until_equal(const uint64_t* flag, uint64_t expect,
                                                 int64_t budget_ticks) {
    if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == expect) return true;
    const uint64_t t0 = wall_clock64();
    for (;;) {
        for (int i = 0; i < 32; ++i) {
            if (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == expect)
                return true;
            __builtin_amdgcn_s_sleep(2);
        }
        if ((int64_t)(wall_clock64() - t0) > budget_ticks) return false;
    }
}

__device__ __forceinline__ void acquire_fence_agent() {
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

__device__ __forceinline__ void report_status(int32_t* status, int code, int a, int b, int c) {
    if (status == nullptr) return;
    // first error wins; plain vector atomics/stores only
    if (atomicCAS(status, SYN_STATUS_OK, code) == SYN_STATUS_OK) {
        status[1] = a;
        status[2] = b;
        status[3] = c;
    }
}

// Hardware workgroup id -> logical program id.  Workgroups are dealt to the
// 8 XCDs round-robin; with the remap each XCD owns a contiguous range of
// logical ids, so the tiles it works on at any moment share A/B panels in
// that XCD's L2.  Identity when remap is off.  A bijection on [0, grid).
__host__ __device__ __forceinline__ int logical_program_id(int hw_id, int grid, bool remap) {
    if (!remap || grid < kNumXcd) return hw_id;
    const int xcd = hw_id % kNumXcd;
    const int slot = hw_id / kNumXcd;
    const int base = grid / kNumXcd;
    const int rem = grid % kNumXcd;
    const int start = xcd * base + (xcd < rem ? xcd : rem);
    return start + slot;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace syn
