// so_conv2d: sparse convolution by implicit im2col on gfx950.
//
// Activations are [C][H][W][B] (batch innermost), so the output of one channel is
// a dense row of H_out*W_out*B columns and the convolution is the same contraction
// as so_matmul with the gathered X row replaced by a shifted window of the input:
// for output column q = (ho, wo, b) and weight column k = (cin, kh, kw) the
// operand is X[cin][ho*sh - ph + kh*dh][wo*sw - pw + kw*dw][b].  Nothing is
// materialised: each lane derives (ho, wo, b) from its column once, the plan holds
// one (offset, dh, dw) triple per stored nonzero, and a tap that falls outside the
// image leaves the accumulator untouched (src/layers/conv.cpp:62-70).  Waves
// whose columns are all interior (the common case) skip the bounds tests.
//
// A workgroup is 8 waves = 8 consecutive output channels on the same columns,
// so the waves of a workgroup gather from the same input window and share it in
// the CU's L1.  Accumulation is bias first, then one fused multiply-add per stored
// nonzero in ascending slot order, as in the reference.
#include "so_internal.h"

#include <cstdlib>
#include <new>

struct so_conv_plan {
    so_conv_geom g;
    const so_ellpack *E = nullptr;
    int2 *d_taps = nullptr;  // per slot: x = (cin*H + dh)*W + dw (elements of B floats), y = dh<<16 | (dw & 0xffff)
};

namespace {

constexpr int kChannelsPerGroup = 8;

template <int VEC> struct ConvVec;
template <> struct ConvVec<1> { using type = float; };
template <> struct ConvVec<2> { using type = float2; };
template <> struct ConvVec<4> { using type = float4; };

template <int VEC>
__device__ __forceinline__ void conv_load(const float *p, float (&v)[VEC])
{
    using T = typename ConvVec<VEC>::type;
    const T t = *reinterpret_cast<const T *>(p);
    if constexpr (VEC == 1) { v[0] = t; }
    if constexpr (VEC == 2) { v[0] = t.x; v[1] = t.y; }
    if constexpr (VEC == 4) { v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
}

// VEC consecutive columns per lane; B % VEC == 0, so a lane's columns belong to
// one output pixel (same taps, same bounds test) and are VEC consecutive batch
// entries: one 4*VEC-byte load per tap.  One batch of 8 taps in flight per wave:
// a second batch in registers was measured slower (the 8 waves of a workgroup
// share the input window through L1 and deeper queues evict it).
template <int VEC, int ACT>
__global__ __launch_bounds__(kChannelsPerGroup * 64)
void conv2d_implicit_kernel(const float *__restrict__ Wd, const int2 *__restrict__ taps,
                            const uint32_t *__restrict__ nnz, uint32_t r, so_conv_geom g,
                            const float *__restrict__ X, uint32_t B, uint64_t ncols,
                            const float *__restrict__ bias, float *__restrict__ Y)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t co = __builtin_amdgcn_readfirstlane(blockIdx.y * kChannelsPerGroup + (threadIdx.x >> 6));
    if (co >= g.Cout) return;
    const uint64_t q = ((uint64_t)blockIdx.x * 64u + lane) * VEC;
    const bool live = q < ncols;
    const uint64_t qq = live ? q : 0;
    const uint32_t p = (uint32_t)(qq / B), b = (uint32_t)(qq % B);
    const int32_t ho = (int32_t)(p / g.W_out), wo = (int32_t)(p % g.W_out);
    const int32_t h0 = ho * (int32_t)g.stride_h - (int32_t)g.pad_h;
    const int32_t w0 = wo * (int32_t)g.stride_w - (int32_t)g.pad_w;
    const int64_t lanebase = ((int64_t)h0 * g.W_in + w0) * (int64_t)B + b;
    const int32_t hspan = (int32_t)((g.kH - 1) * g.dil_h), wspan = (int32_t)((g.kW - 1) * g.dil_w);
    const bool interior = h0 >= 0 && h0 + hspan < (int32_t)g.H_in && w0 >= 0 && w0 + wspan < (int32_t)g.W_in;

    const uint32_t cnt = nnz[co];
    const float *__restrict__ wrow = Wd + (size_t)co * r;
    const int2 *__restrict__ trow = taps + (size_t)co * r;
    float acc[VEC];
    {
        const float b0 = bias ? bias[co] : 0.0f;
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = b0;
    }

    if (__all(interior)) {
        const float *__restrict__ xl = X + lanebase;
        uint32_t j = 0;
        for (; j + 8 <= cnt; j += 8) {
            float w[8], x[8][VEC];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                w[u] = wrow[j + u];
                conv_load<VEC>(xl + (int64_t)trow[j + u].x * (int64_t)B, x[u]);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(w[u], x[u][v], acc[v]);
        }
        for (; j < cnt; ++j) {
            float x[VEC];
            conv_load<VEC>(xl + (int64_t)trow[j].x * (int64_t)B, x);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(wrow[j], x[v], acc[v]);
        }
    } else {
        // Some lane of the wave has taps outside the image.  Same batches of 8, without
        // branches: a tap that is out of bounds for a lane loads a harmless in-bounds
        // address (the lane's own batch entry of pixel (0,0,0)) and contributes
        // fma(w, 0, acc) = acc, which is what skipping it gives.
        const float *__restrict__ xsafe = X + b;
        uint32_t j = 0;
        for (; j + 8 <= cnt; j += 8) {
            float w[8], x[8][VEC];
            bool ok[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int2 t = trow[j + u];
                w[u] = wrow[j + u];
                const int32_t hin = h0 + (t.y >> 16), win = w0 + (int32_t)(int16_t)(t.y & 0xffff);
                ok[u] = (uint32_t)hin < g.H_in && (uint32_t)win < g.W_in;
                conv_load<VEC>(ok[u] ? X + lanebase + (int64_t)t.x * (int64_t)B : xsafe, x[u]);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(w[u], ok[u] ? x[u][v] : 0.0f, acc[v]);
        }
        for (; j < cnt; ++j) {
            const int2 t = trow[j];
            const int32_t hin = h0 + (t.y >> 16), win = w0 + (int32_t)(int16_t)(t.y & 0xffff);
            if ((uint32_t)hin < g.H_in && (uint32_t)win < g.W_in) {
                float x[VEC];
                conv_load<VEC>(X + lanebase + (int64_t)t.x * (int64_t)B, x);
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(wrow[j], x[v], acc[v]);
            }
        }
    }
    if (live) {
        using T = typename ConvVec<VEC>::type;
        T out;
        if constexpr (VEC == 1) { out = so_epilogue<ACT>(acc[0]); }
        if constexpr (VEC == 2) { out.x = so_epilogue<ACT>(acc[0]); out.y = so_epilogue<ACT>(acc[1]); }
        if constexpr (VEC == 4) {
            out.x = so_epilogue<ACT>(acc[0]); out.y = so_epilogue<ACT>(acc[1]);
            out.z = so_epilogue<ACT>(acc[2]); out.w = so_epilogue<ACT>(acc[3]);
        }
        *reinterpret_cast<T *>(Y + (size_t)co * ncols + q) = out;
    }
}

template <int VEC>
void conv_launch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B, uint64_t ncols,
                 const float *dBias, float *dY, int act)
{
    const so_conv_geom &g = plan->g;
    const so_ellpack *E = plan->E;
    const dim3 grid((uint32_t)((ncols + 64ull * VEC - 1) / (64ull * VEC)), so_ceil_div(g.Cout, kChannelsPerGroup));
#define SO_CONV_LAUNCH(A)                                                                          \
    conv2d_implicit_kernel<VEC, A><<<grid, kChannelsPerGroup * 64, 0, ctx->stream>>>(              \
        E->d_Wd, plan->d_taps, E->d_nnz, E->r, g, dX, B, ncols, dBias, dY)
    switch (act) {
    case SO_ACT_RELU:    SO_CONV_LAUNCH(SO_ACT_RELU); break;
    case SO_ACT_SIGMOID: SO_CONV_LAUNCH(SO_ACT_SIGMOID); break;
    case SO_ACT_TANH:    SO_CONV_LAUNCH(SO_ACT_TANH); break;
    default:             SO_CONV_LAUNCH(SO_ACT_NONE); break;
    }
#undef SO_CONV_LAUNCH
}

} // namespace

extern "C" so_status so_conv_plan_create(so_ctx *ctx, const so_ellpack *E, const so_conv_geom *g,
                                         so_conv_plan **out)
{
    SO_REQUIRE(ctx && E && g && out, "so_conv_plan_create: null argument");
    *out = nullptr;
    SO_REQUIRE(g->stride_h && g->stride_w && g->dil_h && g->dil_w && g->kH && g->kW,
               "so_conv_plan_create: kernel size, stride and dilation must be positive");
    SO_REQUIRE(E->m == g->Cout && (uint64_t)E->n == (uint64_t)g->Cin * g->kH * g->kW,
               "so_conv_plan_create: weights are %u x %u, geometry needs %u x %llu", E->m, E->n, g->Cout,
               (unsigned long long)g->Cin * g->kH * g->kW);
    SO_REQUIRE(g->H_in + 2ull * g->pad_h >= (uint64_t)g->dil_h * (g->kH - 1) + 1 &&
               g->W_in + 2ull * g->pad_w >= (uint64_t)g->dil_w * (g->kW - 1) + 1,
               "so_conv_plan_create: kernel window larger than the padded input");
    // Output size as the loader computes it (src/sparse_onnx.cpp:428-429).
    const uint32_t Ho = (g->H_in + 2 * g->pad_h - (g->dil_h * (g->kH - 1) + 1)) / g->stride_h + 1;
    const uint32_t Wo = (g->W_in + 2 * g->pad_w - (g->dil_w * (g->kW - 1) + 1)) / g->stride_w + 1;
    SO_REQUIRE(g->H_out == Ho && g->W_out == Wo, "so_conv_plan_create: H_out x W_out must be %u x %u", Ho, Wo);
    SO_REQUIRE(g->kH * g->dil_h < 32768 && g->kW * g->dil_w < 32768 && g->pad_h < 32768 && g->pad_w < 32768,
               "so_conv_plan_create: kernel extent and padding must be below 32768");
    SO_REQUIRE((uint64_t)g->Cin * g->H_in * g->W_in < (1ull << 31), "so_conv_plan_create: input plane too large");

    const size_t slots = (size_t)E->m * E->r;
    std::vector<uint32_t> idx(slots), nnz(E->m);
    so_status s = so_ellpack_download(ctx, E, SO_LAYOUT_ROW, nullptr, idx.data(), nnz.data());
    if (s != SO_OK) return s;
    std::vector<int2> taps(slots, int2{0, 0});
    const uint32_t kHW = g->kH * g->kW;
    for (uint32_t co = 0; co < E->m; ++co)
        for (uint32_t j = 0; j < nnz[co]; ++j) {
            const uint32_t k = idx[(size_t)co * E->r + j];
            const uint32_t cin = k / kHW, kh = (k / g->kW) % g->kH, kw = k % g->kW;
            const int32_t dh = (int32_t)(kh * g->dil_h), dw = (int32_t)(kw * g->dil_w);
            int2 t;
            t.x = (int32_t)((cin * g->H_in + (uint32_t)dh) * g->W_in + (uint32_t)dw);
            t.y = (dh << 16) | (dw & 0xffff);
            taps[(size_t)co * E->r + j] = t;
        }
    so_conv_plan *plan = new (std::nothrow) so_conv_plan();
    if (!plan) { so_set_error("so_conv_plan_create: host allocation failed"); return SO_ERR_OOM; }
    plan->g = *g;
    plan->E = E;
    void *d = nullptr;
    s = so_malloc(ctx, slots * sizeof(int2), &d);
    if (s == SO_OK) s = so_h2d(ctx, d, taps.data(), slots * sizeof(int2));
    if (s != SO_OK) {
        if (d) (void)hipFree(d);
        delete plan;
        return s;
    }
    plan->d_taps = (int2 *)d;
    *out = plan;
    return SO_OK;
}

extern "C" so_status so_conv_plan_free(so_ctx *ctx, so_conv_plan *plan)
{
    if (!plan) return SO_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (plan->d_taps) (void)hipFree(plan->d_taps);
    delete plan;
    return SO_OK;
}

extern "C" so_status so_conv2d(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                               const float *dBias, float *dY, int act)
{
    SO_REQUIRE(ctx && plan, "so_conv2d: null argument");
    SO_REQUIRE(act >= SO_ACT_NONE && act <= SO_ACT_TANH, "so_conv2d: unknown activation %d", act);
    const so_conv_geom &g = plan->g;
    const uint64_t ncols = (uint64_t)g.H_out * g.W_out * B;
    if (g.Cout == 0 || ncols == 0) return SO_OK;
    SO_REQUIRE(dX && dY, "so_conv2d: null tensor");
    SO_REQUIRE((ncols + 63) / 64 < (1ull << 31), "so_conv2d: output plane too large");
    // Batch entries per lane: as many as divide B and keep 16/8-byte alignment.
    const uintptr_t align = (uintptr_t)dX | (uintptr_t)dY;
    int maxvec = 4;
    if (const char *e = getenv("SPARSEOPS_CONV_VEC")) maxvec = atoi(e);
    if (maxvec >= 4 && B % 4 == 0 && (align & 15) == 0) conv_launch<4>(ctx, plan, dX, B, ncols, dBias, dY, act);
    else if (maxvec >= 2 && B % 2 == 0 && (align & 7) == 0) conv_launch<2>(ctx, plan, dX, B, ncols, dBias, dY, act);
    else conv_launch<1>(ctx, plan, dX, B, ncols, dBias, dY, act);
    SO_LAUNCH_CHECK();
    return SO_OK;
}
