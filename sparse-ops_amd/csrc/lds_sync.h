// Progress counters of a workgroup in LDS, used in place of a barrier per phase by the kernels that
// stream tiles or windows through double-buffered LDS.
//
// The four waves that share a SIMD are served oldest first, and rows differ in length: the waves of
// a workgroup finish a phase up to a third of its length apart, and a barrier makes all of them wait
// for the last one with the SIMDs half idle.  With counters a wave that is done only needs what it
// is about to touch: "every wave has stored its part of the next buffer" before reading it, "every
// wave has finished reading this buffer" before overwriting it.  Stores of the next buffer are made
// half-way through a phase, so a fast wave can run up to half a phase ahead of the slowest.
//
// A wave adds one to a counter when it has stored its part / finished reading; counters only grow
// (targets are 16 waves x the number of times the buffer has been filled / read).  LDS executes a
// wave's operations in order, so the add lands after the wave's stores.  Waits cannot form a cycle:
// every wait is for events of an earlier phase.  The poll nevertheless gives up after kSyncSpins
// tries (a tenth of a second, thousands of launches long), so that no wave can ever hang here; a
// wave that gives up counts itself in g_wait_timeouts, which so_sync() reports as an error.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace so_lds {

constexpr uint32_t kSyncSpins = 1u << 20;
constexpr uint32_t kSyncBytes = 64;      // LDS the counters take (four are used)

// Waits that ran out of tries since the last look (one copy per translation unit that includes this).
static __device__ uint32_t g_wait_timeouts;

// LDS byte address of a pointer into LDS.
__device__ __forceinline__ uint32_t lds_address(const void *p) { return (uint32_t)(uintptr_t)p; }

__device__ __forceinline__ void signal(uint32_t addr, uint32_t lane)
{
    if (lane == 0) asm volatile("ds_add_u32 %0, %1" : : "v"(addr), "v"(1u) : "memory");
}

__device__ __forceinline__ void wait(uint32_t addr, uint32_t target)
{
    for (uint32_t spin = 0; spin < kSyncSpins; ++spin) {
        uint32_t v;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
        if (__builtin_amdgcn_readfirstlane(v) >= target) return;
        __builtin_amdgcn_s_sleep(2);
    }
    if ((threadIdx.x & 63u) == 0) atomicAdd(&g_wait_timeouts, 1u);
}

// Host side: this translation unit's count, set back to zero.
static inline uint32_t take_wait_timeouts()
{
    uint32_t n = 0;
    const uint32_t zero = 0;
    if (hipMemcpyFromSymbol(&n, HIP_SYMBOL(g_wait_timeouts), sizeof n) != hipSuccess) return 0;
    if (n) (void)hipMemcpyToSymbol(HIP_SYMBOL(g_wait_timeouts), &zero, sizeof zero);
    return n;
}

} // namespace so_lds
