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
// wave that gives up counts itself in the context's status word (so_wait_status, passed to the
// kernel), which every entry point that waits for the stream reads and reports as an error.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace so_lds {

constexpr uint32_t kSyncSpins = 1u << 20;
constexpr uint32_t kSyncBytes = 64;      // LDS the counters take (four are used)

// What a kernel needs for its bounded waits: the most polls of one wait (the context's, so that a test
// can make every wait give up at once) and where a wave that gives up counts itself.
struct wait_status {
    uint32_t spins;
    uint32_t *gave_up;
};

// LDS byte address of a pointer into LDS.
__device__ __forceinline__ uint32_t lds_address(const void *p) { return (uint32_t)(uintptr_t)p; }

__device__ __forceinline__ void signal(uint32_t addr, uint32_t lane)
{
    if (lane == 0) asm volatile("ds_add_u32 %0, %1" : : "v"(addr), "v"(1u) : "memory");
}

__device__ __forceinline__ void wait(uint32_t addr, uint32_t target, const wait_status &ws)
{
    for (uint32_t spin = 0; spin < ws.spins; ++spin) {
        uint32_t v;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
        if (__builtin_amdgcn_readfirstlane(v) >= target) return;
        __builtin_amdgcn_s_sleep(2);
    }
    if ((threadIdx.x & 63u) == 0) atomicAdd(ws.gave_up, 1u);
}

} // namespace so_lds
