// Exchange of partial results between workgroups that may sit on different XCDs, whose L2
// caches are not coherent with each other.  Visibility rests on two hardware facts and one
// compiler fact:
//   * a store with device scope (sc1) is written through to memory, and a load with device
//     scope does not take its data from the XCD's L2;
//   * s_waitcnt vmcnt(0) returns when the wave's stores have completed;
//   * the compiler is told not to move memory operations across that wait
//     (__atomic_signal_fence on both sides: relaxed atomics on different addresses could
//     otherwise be reordered around a builtin it knows nothing about).
// No cache write-back or invalidate is issued: those stall every wave of the XCD that is still
// streaming.  16-byte stores written as inline assembly lack the compiler's wait for the
// store data and gave wrong data; the 64-bit atomics below are compiler-visible.
#ifndef YVEX_ROCM_KERNELS_DEVICE_SCOPE_H
#define YVEX_ROCM_KERNELS_DEVICE_SCOPE_H

#include "mfma.h"

__device__ inline void store_b64_device(void *p, float a, float b)
{
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 v = {a, b};
    __hip_atomic_store(reinterpret_cast<uint64_t *>(p), __builtin_bit_cast(uint64_t, v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ inline void load_b64_device(const void *p, float &a, float &b)
{
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 v = __builtin_bit_cast(
        floatx2, __hip_atomic_load(reinterpret_cast<const uint64_t *>(p), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT));
    a = v.x;
    b = v.y;
}

__device__ inline void store_b128_device(void *p, floatx4 v)
{
    store_b64_device(p, v[0], v[1]);
    store_b64_device(reinterpret_cast<float *>(p) + 2, v[2], v[3]);
}

__device__ inline void store_u32x4_device(void *p, u32x4 v)
{
    uint64_t *q = reinterpret_cast<uint64_t *>(p);
    __hip_atomic_store(q, (uint64_t)v.x | ((uint64_t)v.y << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + 1, (uint64_t)v.z | ((uint64_t)v.w << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ inline u32x4 load_u32x4_device(const void *p)
{
    const uint64_t *q = reinterpret_cast<const uint64_t *>(p);
    const uint64_t lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return (u32x4){(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}

// Every store this wave issued so far has completed; nothing moves across.
__device__ inline void stores_completed()
{
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

// Placed between the arrival count that says "the others have published" and the device-scope
// loads of what they published.
__device__ inline void loads_ordered() { __atomic_signal_fence(__ATOMIC_SEQ_CST); }

#endif  // YVEX_ROCM_KERNELS_DEVICE_SCOPE_H
