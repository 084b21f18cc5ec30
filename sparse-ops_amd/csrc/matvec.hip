// so_matvec: y[m] = E * x[n] + bias on gfx950.
//
// The product is a pure stream of the stored (weight, column) pairs -- 8 bytes
// per nonzero and one multiply-add -- so the kernels are built around HBM
// bandwidth: x is staged once per workgroup in LDS when it fits (the gathers
// then never leave the CU), the pairs are read with 16-byte loads, and only the
// first nnz[i] slots of a row are touched, so ELLPACK padding is never streamed.
//
//   wave kernel   one wavefront per row on the row-major arrays; lanes take
//                 aligned groups of four slots, partial sums are combined with a
//                 butterfly of lane exchanges.
//   group kernel  4 or 16 lanes per row, for the short-row classes of a binned
//                 upload (skewed matrices).
//   slot kernel   one lane per row on the slot-major arrays (consecutive rows'
//                 k-th nonzeros are contiguous, so loads coalesce across lanes).
//
// Reference: ellpack_matvec, src/ellpack_matvec.cpp:20-147.  The reference sums
// 16 interleaved partials and a tree (:72-96); the orders here differ, so results
// agree to fp32 round-off, not bit for bit.
#include "so_internal.h"

#include <algorithm>

namespace {

constexpr int kBlock = 512;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int G>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, G);
    return v;
}

// Stage x in LDS (XLDS) or read it through the cache hierarchy.
template <bool XLDS>
__device__ __forceinline__ const float *stage_x(const float *__restrict__ x, uint32_t n, float *lds)
{
    if (!XLDS) return x;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) lds[i] = x[i];
    __syncthreads();
    return lds;
}

// rows == nullptr: row ids are 0..count-1; otherwise the ids come from the list.
template <bool XLDS>
__global__ __launch_bounds__(kBlock)
void matvec_wave_kernel(const float *__restrict__ Wd, const uint32_t *__restrict__ idx,
                        const uint32_t *__restrict__ nnz, const uint32_t *__restrict__ rows,
                        uint32_t count, uint32_t r, const float *__restrict__ x, uint32_t n,
                        const float *__restrict__ bias, float *__restrict__ y)
{
    extern __shared__ float lds_x[];
    const float *xs = stage_x<XLDS>(x, n, lds_x);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = (blockIdx.x * kBlock + threadIdx.x) >> 6;
    const uint32_t nwaves = (gridDim.x * kBlock) >> 6;

    for (uint32_t g = wave; g < count; g += nwaves) {
        const uint32_t row = rows ? rows[g] : g;
        const uint64_t beg = (uint64_t)row * r;
        const uint64_t end = beg + nnz[row];
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        // Aligned groups of four slots covering [beg, end); slots of neighbouring
        // rows that share the first or last group are masked out.
        for (uint64_t q = (beg >> 2) + lane; (q << 2) < end; q += 64) {
            const f32x4 w = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(Wd) + q);
            const u32x4 c = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(idx) + q);
            const uint64_t e = q << 2;
            const bool v0 = e >= beg && e < end, v1 = e + 1 >= beg && e + 1 < end;
            const bool v2 = e + 2 >= beg && e + 2 < end, v3 = e + 3 >= beg && e + 3 < end;
            const float x0 = v0 ? xs[c.x] : 0.0f, x1 = v1 ? xs[c.y] : 0.0f;
            const float x2 = v2 ? xs[c.z] : 0.0f, x3 = v3 ? xs[c.w] : 0.0f;
            a0 = __builtin_fmaf(v0 ? w.x : 0.0f, x0, a0);
            a1 = __builtin_fmaf(v1 ? w.y : 0.0f, x1, a1);
            a2 = __builtin_fmaf(v2 ? w.z : 0.0f, x2, a2);
            a3 = __builtin_fmaf(v3 ? w.w : 0.0f, x3, a3);
        }
        const float s = group_sum<64>((a0 + a1) + (a2 + a3));
        if (lane == 0) y[row] = (bias ? bias[row] : 0.0f) + s;
    }
}

template <int G, bool XLDS>
__global__ __launch_bounds__(kBlock)
void matvec_group_kernel(const float *__restrict__ Wd, const uint32_t *__restrict__ idx,
                         const uint32_t *__restrict__ nnz, const uint32_t *__restrict__ rows,
                         uint32_t count, uint32_t r, const float *__restrict__ x, uint32_t n,
                         const float *__restrict__ bias, float *__restrict__ y)
{
    extern __shared__ float lds_x[];
    const float *xs = stage_x<XLDS>(x, n, lds_x);
    const uint32_t sub = threadIdx.x % G;
    const uint32_t group = (blockIdx.x * kBlock + threadIdx.x) / G;
    const uint32_t ngroups = (gridDim.x * kBlock) / G;

    for (uint32_t g = group; g < count; g += ngroups) {
        const uint32_t row = rows ? rows[g] : g;
        const uint64_t base = (uint64_t)row * r;
        const uint32_t cnt = nnz[row];
        float a = 0.0f;
        for (uint32_t j = sub; j < cnt; j += G)
            a = __builtin_fmaf(Wd[base + j], xs[idx[base + j]], a);
        a = group_sum<G>(a);
        if (sub == 0) y[row] = (bias ? bias[row] : 0.0f) + a;
    }
}

template <bool XLDS>
__global__ __launch_bounds__(kBlock)
void matvec_slot_kernel(const float *__restrict__ WdT, const uint32_t *__restrict__ idxT,
                        const uint32_t *__restrict__ nnz, uint32_t m,
                        const float *__restrict__ x, uint32_t n,
                        const float *__restrict__ bias, float *__restrict__ y)
{
    extern __shared__ float lds_x[];
    const float *xs = stage_x<XLDS>(x, n, lds_x);
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t row = blockIdx.x * kBlock + threadIdx.x; row < m; row += stride) {
        const uint32_t cnt = nnz[row];
        float a = bias ? bias[row] : 0.0f;
        for (uint32_t k = 0; k < cnt; ++k) {
            const size_t e = (size_t)k * m + row;
            a = __builtin_fmaf(WdT[e], xs[idxT[e]], a);
        }
        y[row] = a;
    }
}

// Workgroups to launch for `work` row-units when one workgroup handles `per` of
// them per pass: enough to cover the work, at most a few per compute unit (each
// workgroup re-stages x, so more than that only adds traffic).
uint32_t grid_for(const so_ctx *ctx, uint64_t work, uint32_t per, bool xlds)
{
    const uint32_t need = so_ceil_div(work, per);
    const uint32_t cap = (uint32_t)ctx->compute_units * (xlds ? 2u : 8u);
    return std::max(1u, std::min(need, cap));
}

bool enable_lds(const void *kernel, size_t bytes)
{
    if (bytes <= 48 * 1024) return true;
    return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) == hipSuccess;
}

template <typename K, typename... Args>
so_status launch_x(so_ctx *ctx, K k_lds, K k_gl, uint64_t work, uint32_t per, uint32_t n, Args... args)
{
    const size_t lds = (size_t)n * sizeof(float);
    // x in LDS pays when each workgroup handles many rows; for a handful of rows
    // the staging copy would dominate.
    bool xlds = lds > 0 && lds <= (size_t)ctx->max_lds_bytes && work >= 4ull * per &&
                enable_lds((const void *)k_lds, lds);
    if (!xlds) (void)hipGetLastError();
    const uint32_t blocks = grid_for(ctx, work, per, xlds);
    if (xlds) k_lds<<<blocks, kBlock, lds, ctx->stream>>>(args...);
    else k_gl<<<blocks, kBlock, 0, ctx->stream>>>(args...);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

so_status run_wave(so_ctx *ctx, const so_ellpack *E, const uint32_t *rows, uint32_t count,
                   const float *dx, const float *dBias, float *dy)
{
    return launch_x(ctx, matvec_wave_kernel<true>, matvec_wave_kernel<false>, count, kBlock / 64, E->n,
                    E->d_Wd, E->d_idx, E->d_nnz, rows, count, E->r, dx, E->n, dBias, dy);
}

template <int G>
so_status run_group(so_ctx *ctx, const so_ellpack *E, const uint32_t *rows, uint32_t count,
                    const float *dx, const float *dBias, float *dy)
{
    return launch_x(ctx, matvec_group_kernel<G, true>, matvec_group_kernel<G, false>, count, kBlock / G,
                    E->n, E->d_Wd, E->d_idx, E->d_nnz, rows, count, E->r, dx, E->n, dBias, dy);
}

} // namespace

extern "C" so_status so_matvec(so_ctx *ctx, const so_ellpack *E, const float *dx,
                               const float *dBias, float *dy, int layout)
{
    SO_REQUIRE(ctx && E, "so_matvec: null argument");
    if (E->m == 0) return SO_OK;
    SO_REQUIRE(dy != nullptr, "so_matvec: y is null");
    SO_REQUIRE(dx != nullptr || E->total_nnz == 0, "so_matvec: x is null");
    if (layout == 0) {
        if (E->layouts & SO_LAYOUT_BINS) layout = SO_LAYOUT_BINS;
        else if ((E->layouts & SO_LAYOUT_SLOT) && E->max_nnz <= 64) layout = SO_LAYOUT_SLOT;
        else layout = SO_LAYOUT_ROW;
    }
    SO_REQUIRE(layout == SO_LAYOUT_ROW || layout == SO_LAYOUT_SLOT || layout == SO_LAYOUT_BINS,
               "so_matvec: unknown layout %d", layout);
    SO_REQUIRE((E->layouts & layout) != 0, "so_matvec: layout %d was not uploaded", layout);

    if (layout == SO_LAYOUT_ROW) return run_wave(ctx, E, nullptr, E->m, dx, dBias, dy);
    if (layout == SO_LAYOUT_SLOT)
        return launch_x(ctx, matvec_slot_kernel<true>, matvec_slot_kernel<false>, E->m, kBlock, E->n,
                        E->d_WdT, E->d_idxT, E->d_nnz, E->m, dx, E->n, dBias, dy);
    // Binned: one launch per non-empty length class; every row is in exactly one.
    for (const so_bin &b : E->bins) {
        if (b.count == 0) continue;
        so_status s;
        if (b.group == 4) s = run_group<4>(ctx, E, b.d_rows, b.count, dx, dBias, dy);
        else if (b.group == 16) s = run_group<16>(ctx, E, b.d_rows, b.count, dx, dBias, dy);
        else s = run_wave(ctx, E, b.d_rows, b.count, dx, dBias, dy);
        if (s != SO_OK) return s;
    }
    return SO_OK;
}
