// Steps of a sparse row fed from LDS, with the row's (weight, LDS byte offset) pairs held one per
// lane and handed round by DPP: lane N of every 16-lane row holds step N's pair (all four rows of
// the wave may hold different pairs, or the same ones), `row_newbcast:N` broadcasts it inside its
// row.  One step = one 16-byte LDS read + four multiply-adds into the lane's four accumulators;
// the weight's broadcast rides on the multiply-add (v_fmac_f32_dpp), the offset's on the address
// add.  Steps run in order, so each accumulator sees its products in step order.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace so_dpp {

template <int N>
__device__ __forceinline__ float bcast_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x150 + N, 0xf, 0xf, true));
}
template <int N>
__device__ __forceinline__ uint32_t bcast_u(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x150 + N, 0xf, 0xf, true);
}

template <int N>
__device__ __forceinline__ void fmac_bcast(float &acc, float ew, float x)
{
    asm("v_fmac_f32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(ew), "v"(x), "n"(N));
}

// Steps N..END-1 of a chunk: all LDS reads first, then the FMAs in step order.
template <int N, int END>
struct StepRange {
    static __device__ __forceinline__ void read(const char *base, uint32_t eoff, float4 *x)
    {
        x[0] = *reinterpret_cast<const float4 *>(base + bcast_u<N>(eoff));
        StepRange<N + 1, END>::read(base, eoff, x + 1);
    }
    static __device__ __forceinline__ void fma(float ew, const float4 *x, float (&acc)[4])
    {
        // acc += bcast(ew) * x with the broadcast folded into the multiply-add's first operand
        // (v_fmac_f32 is a fused multiply-add: one rounding, like fmaf)
        fmac_bcast<N>(acc[0], ew, x[0].x);
        fmac_bcast<N>(acc[1], ew, x[0].y);
        fmac_bcast<N>(acc[2], ew, x[0].z);
        fmac_bcast<N>(acc[3], ew, x[0].w);
        StepRange<N + 1, END>::fma(ew, x + 1, acc);
    }
};
template <int END>
struct StepRange<END, END> {
    static __device__ __forceinline__ void read(const char *, uint32_t, float4 *) {}
    static __device__ __forceinline__ void fma(float, const float4 *, float (&)[4]) {}
};

template <int N0, int CNT>
__device__ __forceinline__ void tiled_steps(const char *base, float ew, uint32_t eoff, float (&acc)[4])
{
    float4 x[CNT];
    StepRange<N0, N0 + CNT>::read(base, eoff, x);
    // a DPP operand must not be read within two cycles of a vector write to it, nor within five of
    // a vector write to the execution mask; the compiler does not see inside the asm
    asm volatile("s_nop 4" : "+v"(ew));
    StepRange<N0, N0 + CNT>::fma(ew, x, acc);
}

// One chunk; `left` = steps still to do in this tile (a positive multiple of 4).
__device__ __forceinline__ void tiled_chunk(const char *base, float ew, uint32_t eoff, uint32_t left, float (&acc)[4])
{
    if (left >= 8) {
        tiled_steps<0, 8>(base, ew, eoff, acc);
        if (left >= 16) tiled_steps<8, 8>(base, ew, eoff, acc);
        else if (left >= 12) tiled_steps<8, 4>(base, ew, eoff, acc);
    } else {
        tiled_steps<0, 4>(base, ew, eoff, acc);
    }
}

// ---- the same steps, software-pipelined ------------------------------------------------
//
// Four steps (a quad) at a time: the quad's four LDS reads go out, and while they are in flight the
// previous quad's sixteen multiply-adds run on operands that have already arrived.  LDS returns data
// in order, so the wait in front of a quad's multiply-adds leaves the next quad's four reads in
// flight.  Two operand buffers, A and B; between groups of sixteen steps the quad still owed its
// multiply-adds sits in B.  The scheduling fences keep the compiler from moving a quad's
// multiply-adds back in front of the reads that are meant to overlap them.  One straight-line body
// per group length: a branch around reads would make the compiler's wait counts assume the path with
// the fewest reads in flight, which turns every later wait into a full one.
template <int N0>
__device__ __forceinline__ void quad_read(const char *base, uint32_t eoff, float4 (&x)[4])
{
    StepRange<N0, N0 + 4>::read(base, eoff, x);
    __builtin_amdgcn_sched_barrier(0);
}
template <int N0>
__device__ __forceinline__ void quad_fma(float ew, const float4 (&x)[4], float (&acc)[4])
{
    StepRange<N0, N0 + 4>::fma(ew, x, acc);
    __builtin_amdgcn_sched_barrier(0);
}

// A full group of sixteen steps.  OWED: quad 3 of the previous group (pairs in ewp, operands in xB)
// still has its multiply-adds to do.  Leaves this group's quad 3 owed, operands in xB.
template <bool OWED>
__device__ __forceinline__ void group16(const char *base, float ew, uint32_t eoff, float ewp, float4 (&xA)[4], float4 (&xB)[4],
                                        float (&acc)[4])
{
    asm volatile("s_nop 4" : "+v"(ew), "+v"(eoff));       // DPP operands: not within two cycles of a vector write
    quad_read<0>(base, eoff, xA);
    if constexpr (OWED) quad_fma<12>(ewp, xB, acc);
    quad_read<4>(base, eoff, xB);
    quad_fma<0>(ew, xA, acc);
    quad_read<8>(base, eoff, xA);
    quad_fma<4>(ew, xB, acc);
    quad_read<12>(base, eoff, xB);
    quad_fma<8>(ew, xA, acc);
}

// The last group of a run: `quads` (1..3) quads, then nothing is owed any more.
template <bool OWED>
__device__ __forceinline__ void group_tail(uint32_t quads, const char *base, float ew, uint32_t eoff, float ewp, float4 (&xA)[4],
                                           float4 (&xB)[4], float (&acc)[4])
{
    asm volatile("s_nop 4" : "+v"(ew), "+v"(eoff));
    quad_read<0>(base, eoff, xA);
    if constexpr (OWED) quad_fma<12>(ewp, xB, acc);
    if (quads == 1u) {
        quad_fma<0>(ew, xA, acc);
    } else {
        quad_read<4>(base, eoff, xB);
        quad_fma<0>(ew, xA, acc);
        if (quads == 2u) {
            quad_fma<4>(ew, xB, acc);
        } else {
            quad_read<8>(base, eoff, xA);
            quad_fma<4>(ew, xB, acc);
            quad_fma<8>(ew, xA, acc);
        }
    }
}

// The multiply-adds still owed after a run's last full group.
__device__ __forceinline__ void group_drain(float ewp, const float4 (&xB)[4], float (&acc)[4])
{
    asm volatile("s_nop 1" : "+v"(ewp));
    quad_fma<12>(ewp, xB, acc);
}

} // namespace so_dpp
