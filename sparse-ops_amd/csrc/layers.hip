// Bandwidth-bound layer kernels of the model chain: max-pool, global average
// pool, elementwise add, stand-alone activations and the 2-D transpose used at
// the host boundary.  All tensors are [C][H][W][B] / [features][B], batch innermost,
// so consecutive lanes always touch consecutive addresses.
#include "so_internal.h"

#include <algorithm>

namespace {

constexpr int kBlock = 256;

// applyMaxPool (src/layers/pool.cpp:28-101): -inf start, taps outside the image skipped.
__global__ __launch_bounds__(kBlock)
void maxpool_kernel(so_pool_geom p, const float *__restrict__ X, uint32_t B, uint64_t total,
                    float *__restrict__ Y)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t q = (uint64_t)blockIdx.x * kBlock + threadIdx.x; q < total; q += stride) {
        const uint32_t b = (uint32_t)(q % B);
        uint64_t t = q / B;
        const uint32_t wo = (uint32_t)(t % p.W_out); t /= p.W_out;
        const uint32_t ho = (uint32_t)(t % p.H_out);
        const uint32_t c = (uint32_t)(t / p.H_out);
        const int32_t h0 = (int32_t)ho * p.sH - p.padH0, w0 = (int32_t)wo * p.sW - p.padW0;
        float v = -INFINITY;
        for (int32_t kh = 0; kh < p.kH; ++kh) {
            const int32_t hin = h0 + kh;
            if ((uint32_t)hin >= p.H) continue;
            for (int32_t kw = 0; kw < p.kW; ++kw) {
                const int32_t win = w0 + kw;
                if ((uint32_t)win >= p.W) continue;
                const float x = X[(((uint64_t)c * p.H + (uint32_t)hin) * p.W + (uint32_t)win) * B + b];
                v = x > v ? x : v;
            }
        }
        Y[q] = v;
    }
}

// The same with four batch entries per lane (B % 4 == 0, 16-byte aligned tensors): one 16-byte
// load per tap, 32-bit index arithmetic.  Per component the comparisons run in the same order.
__global__ __launch_bounds__(kBlock)
void maxpool4_kernel(so_pool_geom p, const float *__restrict__ X, uint32_t B4, uint32_t total,
                     float *__restrict__ Y)
{
    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD one contiguous eighth of the
    // output instead, so that the input rows two neighbouring output rows share meet in one L2.
    const uint32_t per_xcd = gridDim.x / 8u;                     // the grid is a multiple of 8
    const uint32_t vblock = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    const uint32_t chunk = (total + 8u * per_xcd - 1u) / (8u * per_xcd);        // outputs per workgroup
    const uint32_t q_end = min(total, (vblock + 1u) * chunk);
    for (uint32_t q = vblock * chunk + threadIdx.x; q < q_end; q += kBlock) {
        const uint32_t b = q % B4;
        uint32_t t = q / B4;
        const uint32_t wo = t % p.W_out; t /= p.W_out;
        const uint32_t ho = t % p.H_out;
        const uint32_t c = t / p.H_out;
        const int32_t h0 = (int32_t)ho * p.sH - p.padH0, w0 = (int32_t)wo * p.sW - p.padW0;
        float4 v = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        const float4 *__restrict__ Xc = reinterpret_cast<const float4 *>(X) + (size_t)c * p.H * p.W * B4 + b;
        for (int32_t kh = 0; kh < p.kH; ++kh) {
            const int32_t hin = h0 + kh;
            if ((uint32_t)hin >= p.H) continue;
            for (int32_t kw = 0; kw < p.kW; ++kw) {
                const int32_t win = w0 + kw;
                if ((uint32_t)win >= p.W) continue;
                const float4 x = Xc[((uint32_t)hin * p.W + (uint32_t)win) * B4];
                v.x = x.x > v.x ? x.x : v.x;
                v.y = x.y > v.y ? x.y : v.y;
                v.z = x.z > v.z ? x.z : v.z;
                v.w = x.w > v.w ? x.w : v.w;
            }
        }
        reinterpret_cast<float4 *>(Y)[q] = v;
    }
}

// applyGlobalAveragePool (src/layers/pool.cpp:103-154): fp32 running sum over h
// then w, times 1.0f/float(H*W).  One lane per (c, b).
__global__ __launch_bounds__(kBlock)
void gap_kernel(uint32_t C, uint32_t HW, const float *__restrict__ X, uint32_t B, float scale,
                float *__restrict__ Y)
{
    const uint64_t total = (uint64_t)C * B;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t q = (uint64_t)blockIdx.x * kBlock + threadIdx.x; q < total; q += stride) {
        const uint32_t b = (uint32_t)(q % B);
        const uint64_t c = q / B;
        const float *xp = X + c * HW * B + b;
        float s = 0.0f;
        uint32_t i = 0;
        for (; i + 8 <= HW; i += 8) {            // eight loads in flight, the additions still in order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = xp[(uint64_t)(i + u) * B];
#pragma unroll
            for (int u = 0; u < 8; ++u) s = s + v[u];
        }
        for (; i < HW; ++i) s = s + xp[(uint64_t)i * B];
        Y[q] = s * scale;
    }
}

// applyAdd (src/layers/add.cpp:9-76).  D may be A or B.  Aligned operands: 16 bytes per lane, chunks of 16 KB per
// workgroup and operand, all eight loads of a lane requested before the first sum, non-temporal stores.
__global__ __launch_bounds__(kBlock)
void add_kernel(const float *A, const float *Bv, size_t len, float *D)
{
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int U = 4;
    constexpr size_t kChunk = (size_t)U * kBlock;
    size_t done = 0;
    if ((((uintptr_t)A | (uintptr_t)Bv | (uintptr_t)D) & 15u) == 0) {
        const size_t nchunks = len / (4 * kChunk);
        const f4 *A4 = reinterpret_cast<const f4 *>(A), *B4 = reinterpret_cast<const f4 *>(Bv);
        f4 *D4 = reinterpret_cast<f4 *>(D);
        for (size_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
            const size_t i = c * kChunk + threadIdx.x;
            f4 a[U], b[U];
#pragma unroll
            for (int u = 0; u < U; ++u) { a[u] = A4[i + (size_t)u * kBlock]; b[u] = B4[i + (size_t)u * kBlock]; }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                f4 r;
                r[0] = a[u][0] + b[u][0]; r[1] = a[u][1] + b[u][1]; r[2] = a[u][2] + b[u][2]; r[3] = a[u][3] + b[u][3];
                __builtin_nontemporal_store(r, D4 + i + (size_t)u * kBlock);
            }
        }
        done = nchunks * 4 * kChunk;
    }
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = done + (size_t)blockIdx.x * kBlock + threadIdx.x; i < len; i += stride) D[i] = A[i] + Bv[i];
}

// Streams X through the activation into Y (Y may be X).  Aligned operands go in chunks of 32 KB per workgroup:
// 16 bytes per lane, kCopyUnroll loads requested before the first result is used, stores non-temporal (the
// result is not read again by this kernel).  STREAM: operands larger than the 256 MB Infinity Cache -- the loads
// are non-temporal too and a chunk takes two trips of four loads; otherwise one trip of eight plain loads (a
// source that an earlier launch left in the cache is then served from there).  Measured, 256 MiB in + out:
// 4.8 TB/s with one float per lane and a grid-stride loop, 8.4 in this form; 1 GiB in + out: 6.3 TB/s
// (79 % of the HBM peak; plain loads 5.6).
constexpr int kCopyUnroll = 8;
constexpr size_t kCopyChunk = (size_t)kCopyUnroll * kBlock;      // 16-byte elements per workgroup
template <int ACT, bool STREAM>
__global__ __launch_bounds__(kBlock)
void act_kernel(const float *X, size_t len, float *Y)
{
    typedef float f4 __attribute__((ext_vector_type(4)));
    constexpr int U = STREAM ? kCopyUnroll / 2 : kCopyUnroll;
    size_t done = 0;
    if ((((uintptr_t)X | (uintptr_t)Y) & 15u) == 0) {
        const size_t nchunks = len / (4 * kCopyChunk);
        const f4 *X4 = reinterpret_cast<const f4 *>(X);
        f4 *Y4 = reinterpret_cast<f4 *>(Y);
        for (size_t c = blockIdx.x; c < nchunks; c += gridDim.x) {
#pragma unroll
            for (int h = 0; h < kCopyUnroll / U; ++h) {
                const size_t i = c * kCopyChunk + (size_t)h * U * kBlock + threadIdx.x;
                f4 v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = STREAM ? __builtin_nontemporal_load(X4 + i + (size_t)u * kBlock) : X4[i + (size_t)u * kBlock];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    f4 r;
                    r[0] = so_epilogue<ACT>(v[u][0]); r[1] = so_epilogue<ACT>(v[u][1]); r[2] = so_epilogue<ACT>(v[u][2]); r[3] = so_epilogue<ACT>(v[u][3]);
                    __builtin_nontemporal_store(r, Y4 + i + (size_t)u * kBlock);
                }
            }
        }
        done = nchunks * 4 * kCopyChunk;
    }
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = done + (size_t)blockIdx.x * kBlock + threadIdx.x; i < len; i += stride) Y[i] = so_epilogue<ACT>(X[i]);
}

// 64x64 tiles through LDS (+1 padding against bank conflicts): both the read of
// src rows and the write of dst rows are coalesced.
__global__ __launch_bounds__(kBlock)
void transpose_kernel(const float *__restrict__ src, uint32_t rows, uint32_t cols, float *__restrict__ dst)
{
    __shared__ float tile[64][65];
    const uint32_t tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;  // 64 x 4
    const uint32_t r0 = blockIdx.y * 64u, c0 = blockIdx.x * 64u;
    for (uint32_t i = ty; i < 64; i += 4)
        if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = src[(size_t)(r0 + i) * cols + c0 + tx];
    __syncthreads();
    for (uint32_t i = ty; i < 64; i += 4)
        if (c0 + i < cols && r0 + tx < rows) dst[(size_t)(c0 + i) * rows + r0 + tx] = tile[tx][i];
}

// dst[i2][i1][i0][:] = src[i0][i1][i2][:], rows of `inner` floats.  A lane per destination float:
// writes are contiguous, reads come in runs of `inner` floats.
__global__ __launch_bounds__(kBlock)
void reverse_axes3_kernel(const float *__restrict__ src, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t inner,
                          float *__restrict__ dst, size_t total)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t o = (size_t)blockIdx.x * kBlock + threadIdx.x; o < total; o += stride) {
        const uint32_t e = (uint32_t)(o % inner);
        size_t t = o / inner;
        const uint32_t i0 = (uint32_t)(t % d0);
        t /= d0;
        const uint32_t i1 = (uint32_t)(t % d1), i2 = (uint32_t)(t / d1);
        dst[o] = src[(((size_t)i0 * d1 + i1) * d2 + i2) * inner + e];
    }
}

uint32_t blocks_for(const so_ctx *ctx, uint64_t work)
{
    const uint64_t need = (work + kBlock - 1) / kBlock;
    return (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>(need, (uint64_t)ctx->compute_units * 16));
}

} // namespace

extern "C" so_status so_maxpool(so_ctx *ctx, const so_pool_geom *p, const float *dX, uint32_t B, float *dY)
{
    SO_REQUIRE(ctx && p, "so_maxpool: null argument");
    SO_REQUIRE(p->kH > 0 && p->kW > 0 && p->sH > 0 && p->sW > 0 && p->padH0 >= 0 && p->padW0 >= 0,
               "so_maxpool: kernel and stride must be positive, pads non-negative");
    const uint64_t total = (uint64_t)p->C * p->H_out * p->W_out * B;
    if (total == 0) return SO_OK;
    SO_REQUIRE(dX && dY, "so_maxpool: null tensor");
    // Every output window must start inside the padded image.
    SO_REQUIRE((uint64_t)(p->H_out - 1) * p->sH < (uint64_t)p->H + p->padH0 &&
               (uint64_t)(p->W_out - 1) * p->sW < (uint64_t)p->W + p->padW0,
               "so_maxpool: output size does not fit the input");
    if (B % 4 == 0 && (((uintptr_t)dX | (uintptr_t)dY) & 15) == 0 && total / 4 < (1ull << 31) &&
        (uint64_t)p->H * p->W * (B / 4) < (1ull << 31))
        maxpool4_kernel<<<(blocks_for(ctx, total / 4) + 7u) / 8u * 8u, kBlock, 0, ctx->stream>>>(*p, dX, B / 4, (uint32_t)(total / 4), dY);   // a multiple of 8: the kernel deals whole eighths to the XCDs
    else
        maxpool_kernel<<<blocks_for(ctx, total), kBlock, 0, ctx->stream>>>(*p, dX, B, total, dY);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_gap(so_ctx *ctx, uint32_t C, uint32_t H, uint32_t W, const float *dX,
                            uint32_t B, float *dY)
{
    SO_REQUIRE(ctx != nullptr, "so_gap: ctx is null");
    const uint64_t total = (uint64_t)C * B;
    if (total == 0) return SO_OK;
    SO_REQUIRE(dX && dY && H && W, "so_gap: null tensor or empty plane");
    const float scale = 1.0f / (float)(H * W);
    gap_kernel<<<blocks_for(ctx, total), kBlock, 0, ctx->stream>>>(C, H * W, dX, B, scale, dY);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_add(so_ctx *ctx, const float *dA, const float *dB, size_t len, float *dD)
{
    SO_REQUIRE(ctx != nullptr, "so_add: ctx is null");
    if (len == 0) return SO_OK;
    SO_REQUIRE(dA && dB && dD, "so_add: null tensor");
    // one workgroup per 16 KB chunk of each operand
    const uint32_t blocks = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>((len + 4095) / 4096, 1u << 20));
    add_kernel<<<blocks, kBlock, 0, ctx->stream>>>(dA, dB, len, dD);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_act(so_ctx *ctx, int act, const float *dX, size_t len, float *dY)
{
    SO_REQUIRE(ctx != nullptr, "so_act: ctx is null");
    SO_REQUIRE(act >= SO_ACT_NONE && act <= SO_ACT_TANH, "so_act: unknown activation %d", act);
    if (len == 0) return SO_OK;
    SO_REQUIRE(dX && dY, "so_act: null tensor");
    // one workgroup per 32 KB chunk
    const uint32_t blocks = (uint32_t)std::max<uint64_t>(1, std::min<uint64_t>((len + 4 * kCopyChunk - 1) / (4 * kCopyChunk), 1u << 20));
    const bool stream = (uint64_t)len * 8 > (256ull << 20);          // source and result together do not fit the Infinity Cache
#define SO_ACT_LAUNCH(A)                                                                          \
    do {                                                                                          \
        if (stream) act_kernel<A, true><<<blocks, kBlock, 0, ctx->stream>>>(dX, len, dY);         \
        else act_kernel<A, false><<<blocks, kBlock, 0, ctx->stream>>>(dX, len, dY);               \
    } while (0)
    switch (act) {
    case SO_ACT_RELU:    SO_ACT_LAUNCH(SO_ACT_RELU); break;
    case SO_ACT_SIGMOID: SO_ACT_LAUNCH(SO_ACT_SIGMOID); break;
    case SO_ACT_TANH:    SO_ACT_LAUNCH(SO_ACT_TANH); break;
    default:             SO_ACT_LAUNCH(SO_ACT_NONE); break;
    }
#undef SO_ACT_LAUNCH
    SO_LAUNCH_CHECK();
    return SO_OK;
}

// dst row i = src row i's first `cols` values, then zeros up to dst_stride (src_stride, dst_stride in floats).
__global__ __launch_bounds__(kBlock)
void copy_rows_kernel(const float *__restrict__ src, size_t src_stride, uint32_t cols, float *__restrict__ dst,
                      size_t dst_stride, uint32_t dst_cols, size_t total)
{
    for (size_t e = (size_t)blockIdx.x * kBlock + threadIdx.x; e < total; e += (size_t)gridDim.x * kBlock) {
        const size_t row = e / dst_cols;
        const uint32_t c = (uint32_t)(e % dst_cols);
        dst[row * dst_stride + c] = c < cols ? src[row * src_stride + c] : 0.0f;
    }
}

extern "C" so_status so_copy_rows(so_ctx *ctx, const float *dSrc, size_t src_stride, uint32_t rows, uint32_t cols,
                                  float *dDst, size_t dst_stride, int zero_fill)
{
    SO_REQUIRE(ctx != nullptr, "so_copy_rows: ctx is null");
    if (rows == 0 || cols == 0) return SO_OK;
    SO_REQUIRE(dSrc && dDst, "so_copy_rows: null tensor");
    SO_REQUIRE(src_stride >= cols && dst_stride >= cols, "so_copy_rows: a stride is shorter than a row");
    const uint32_t dst_cols = zero_fill ? (uint32_t)std::min<size_t>(dst_stride, 0xffffffffu) : cols;
    const size_t total = (size_t)rows * dst_cols;
    copy_rows_kernel<<<blocks_for(ctx, total), kBlock, 0, ctx->stream>>>(dSrc, src_stride, cols, dDst, dst_stride, dst_cols, total);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_transpose(so_ctx *ctx, const float *dSrc, uint32_t rows, uint32_t cols, float *dDst)
{
    SO_REQUIRE(ctx != nullptr, "so_transpose: ctx is null");
    if (rows == 0 || cols == 0) return SO_OK;
    SO_REQUIRE(dSrc && dDst && dSrc != dDst, "so_transpose: null or aliased tensor");
    const dim3 grid(so_ceil_div(cols, 64), so_ceil_div(rows, 64));
    SO_REQUIRE(grid.y < 65536, "so_transpose: too many rows");
    transpose_kernel<<<grid, kBlock, 0, ctx->stream>>>(dSrc, rows, cols, dDst);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_reverse_axes3(so_ctx *ctx, const float *dSrc, uint32_t d0, uint32_t d1, uint32_t d2, uint32_t inner,
                                      float *dDst)
{
    SO_REQUIRE(ctx != nullptr, "so_reverse_axes3: ctx is null");
    const size_t total = (size_t)d0 * d1 * d2 * inner;
    if (total == 0) return SO_OK;
    SO_REQUIRE(dSrc && dDst && dSrc != dDst, "so_reverse_axes3: null or aliased tensor");
    reverse_axes3_kernel<<<blocks_for(ctx, total), kBlock, 0, ctx->stream>>>(dSrc, d0, d1, d2, inner, dDst, total);
    SO_LAUNCH_CHECK();
    return SO_OK;
}
