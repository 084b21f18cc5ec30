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

} // namespace so_dpp
