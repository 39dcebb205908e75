// Partial-result slots exchanged between workgroups: a 16-byte slot holds four fp32 values or the
// sentinel 0xFFFFFFFF ("empty") in every word.  Validity travels with each 32-bit value, so the
// accesses need no fences; they are agent-scope relaxed atomics (served at the device coherence
// point, never stale in a CU's L1).
#pragma once

#include "common.h"

namespace w4a16 {

constexpr uint32_t kEmpty = 0xFFFFFFFFu;
#ifndef POLL_SLEEP
#define POLL_SLEEP 1   // s_sleep units of 64 cycles between issuing the two polling rounds (0..2 measure the same, 8 and 16 slower)
#endif

// 16-byte slot access as two 8-byte atomics.
#ifndef SLOT_ST_SCOPE
#define SLOT_ST_SCOPE __HIP_MEMORY_SCOPE_AGENT
#endif
#ifndef SLOT_LD_SCOPE
#define SLOT_LD_SCOPE __HIP_MEMORY_SCOPE_AGENT
#endif
__device__ __forceinline__ void slot_store(float *p, u32x4 v) {
    uint64_t *q = reinterpret_cast<uint64_t *>(p);
    __hip_atomic_store(q, (uint64_t)v[0] | ((uint64_t)v[1] << 32), __ATOMIC_RELAXED, SLOT_ST_SCOPE);
    __hip_atomic_store(q + 1, (uint64_t)v[2] | ((uint64_t)v[3] << 32), __ATOMIC_RELAXED, SLOT_ST_SCOPE);
}
__device__ __forceinline__ u32x4 slot_load(const float *p) {
    const uint64_t *q = reinterpret_cast<const uint64_t *>(p);
    const uint64_t a = __hip_atomic_load(q, __ATOMIC_RELAXED, SLOT_LD_SCOPE);
    const uint64_t b = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, SLOT_LD_SCOPE);
    return u32x4{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
}
// The same slot split over two planes `plane` floats apart: thread e keeps words 0, 1 at pa and words 2, 3 at
// pa + plane, with pa = base + 2 e.  Each of the two 8-byte accesses of a wavefront then covers 512 contiguous
// bytes (the interleaved form writes every 32-byte sector twice, half of it each time).
__device__ __forceinline__ void slot_store_planes(float *pa, size_t plane, u32x4 v) {
    __hip_atomic_store(reinterpret_cast<uint64_t *>(pa), (uint64_t)v[0] | ((uint64_t)v[1] << 32), __ATOMIC_RELAXED, SLOT_ST_SCOPE);
    __hip_atomic_store(reinterpret_cast<uint64_t *>(pa + plane), (uint64_t)v[2] | ((uint64_t)v[3] << 32), __ATOMIC_RELAXED, SLOT_ST_SCOPE);
}
__device__ __forceinline__ u32x4 slot_load_planes(const float *pa, size_t plane) {
    const uint64_t a = __hip_atomic_load(reinterpret_cast<const uint64_t *>(pa), __ATOMIC_RELAXED, SLOT_LD_SCOPE);
    const uint64_t b = __hip_atomic_load(reinterpret_cast<const uint64_t *>(pa + plane), __ATOMIC_RELAXED, SLOT_LD_SCOPE);
    return u32x4{(uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32)};
}
__device__ __forceinline__ bool slot_full(u32x4 v) {
    return v[0] != kEmpty && v[1] != kEmpty && v[2] != kEmpty && v[3] != kEmpty;
}

}  // namespace w4a16
