// so_matvec: y[m] = E * x[n] + bias on gfx950.
//
// The product is a pure stream of the stored (weight, column) pairs -- 8 bytes
// per nonzero and one multiply-add -- so the kernels are built around HBM
// bandwidth: x is staged once per workgroup in LDS when it fits (the gathers
// then never leave the CU), the pairs are read with 16-byte non-temporal loads,
// four per lane in flight, and only the first nnz[i] slots of a row are touched,
// so ELLPACK padding is never streamed.  A handle uploaded with SO_LAYOUT_IDX16 also has
// its columns in 16 bits: the kernels then stream 6 bytes per nonzero.
//
//   rows kernel    one wavefront per row on the row-major arrays; lanes take
//                  aligned groups of four slots, partial sums are combined with a
//                  butterfly of lane exchanges.
//   binned kernel  one launch over four length classes (skewed matrices): a whole
//                  workgroup for rows of more than 4096 nonzeros, whole waves for
//                  long rows, 16 or 4 lanes per row for short ones; workgroups of
//                  the long classes are dispatched first.
//   slot kernel    one lane per row on the slot-major arrays (consecutive rows'
//                  k-th nonzeros are contiguous, so loads coalesce across lanes).
//
// Reference: ellpack_matvec, src/ellpack_matvec.cpp:20-147.  The reference sums
// 16 interleaved partials and a tree (:72-96); the orders here differ, so results
// agree to fp32 round-off, not bit for bit.
#include "so_internal.h"

#include <algorithm>

namespace {

constexpr int kBlock = 1024;
constexpr int kWavesPerBlock = kBlock / 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// The columns of four consecutive slots as they are loaded: four 32-bit words, or two when the
// handle carries its columns in 16 bits as well (SO_LAYOUT_IDX16: 6 bytes per nonzero instead of 8).
template <bool I16> struct ColGroup;
template <> struct ColGroup<false> {
    using T = u32x4;
    using E = uint32_t;
    static __device__ __forceinline__ u32x4 cols(T t) { return t; }
};
template <> struct ColGroup<true> {
    using T = u32x2;
    using E = uint16_t;
    static __device__ __forceinline__ u32x4 cols(T t)
    {
        u32x4 c;
        c.x = t.x & 0xffffu; c.y = t.x >> 16; c.z = t.y & 0xffffu; c.w = t.y >> 16;
        return c;
    }
};

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
    const uint32_t n4 = ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) ? n / 4 : 0;     // 16-byte copies when x is aligned
    for (uint32_t i = threadIdx.x; i < n4; i += blockDim.x)
        reinterpret_cast<float4 *>(lds)[i] = reinterpret_cast<const float4 *>(x)[i];
    for (uint32_t i = n4 * 4 + threadIdx.x; i < n; i += blockDim.x) lds[i] = x[i];
    __syncthreads();
    return lds;
}

// Dot product of one row with x, computed by a whole wave, in two halves so that a caller can
// put other work (staging x, finishing the previous row) between issuing the loads and using
// them.  The row's slots [beg, end) are covered by aligned groups of four; a lane loads up to four
// such groups (addresses past the row are clamped onto its last group and every slot outside
// [beg, end) is masked to an exact no-op).  Rows longer than 1024 slots continue in row_rest.
template <bool I16>
struct RowLoads {
    f32x4 w[4];
    typename ColGroup<I16>::T c[4];
};

// G = lanes that share a row (64, 32, 16 or 8): a pass of the row covers 16 G slots.
template <int G, bool I16>
__device__ __forceinline__ void row_issue(const f32x4 *__restrict__ Wd4, const typename ColGroup<I16>::T *__restrict__ idx4,
                                          uint64_t beg, uint64_t end, uint64_t q0, RowLoads<I16> &L)
{
    const uint64_t qlast = end > beg ? (end - 1) >> 2 : beg >> 2;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const uint64_t q = std::min<uint64_t>(q0 + (uint64_t)G * u, qlast);
        L.w[u] = __builtin_nontemporal_load(Wd4 + q);
        L.c[u] = __builtin_nontemporal_load(idx4 + q);
    }
}

template <int G, bool I16>
__device__ __forceinline__ void row_consume(const RowLoads<I16> &L, uint64_t beg, uint64_t end, uint64_t q0, const float *xs,
                                            float &a0, float &a1, float &a2, float &a3)
{
    // slot k of group u is live iff its distance from the row's start is in [0, end - beg): one
    // unsigned 32-bit comparison (a slot before the row gives a huge distance)
    const uint32_t len = (uint32_t)(end - beg);
    const int32_t rel0 = (int32_t)(int64_t)((q0 << 2) - beg);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int32_t rel = rel0 + 4 * G * u;
        const bool v0 = (uint32_t)rel < len, v1 = (uint32_t)(rel + 1) < len;
        const bool v2 = (uint32_t)(rel + 2) < len, v3 = (uint32_t)(rel + 3) < len;
        const u32x4 c = ColGroup<I16>::cols(L.c[u]);
        const float x0 = xs[v0 ? c.x : 0u], x1 = xs[v1 ? c.y : 0u];
        const float x2 = xs[v2 ? c.z : 0u], x3 = xs[v3 ? c.w : 0u];
        a0 = __builtin_fmaf(v0 ? L.w[u].x : 0.0f, v0 ? x0 : 0.0f, a0);
        a1 = __builtin_fmaf(v1 ? L.w[u].y : 0.0f, v1 ? x1 : 0.0f, a1);
        a2 = __builtin_fmaf(v2 ? L.w[u].z : 0.0f, v2 ? x2 : 0.0f, a2);
        a3 = __builtin_fmaf(v3 ? L.w[u].w : 0.0f, v3 ? x3 : 0.0f, a3);
    }
}

// The whole row at once (used where rows are not pipelined).
template <bool I16>
__device__ __forceinline__ float wave_row_dot(const f32x4 *__restrict__ Wd4, const typename ColGroup<I16>::T *__restrict__ idx4,
                                              uint64_t beg, uint64_t end, const float *xs, uint32_t lane)
{
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    if (end == beg) return 0.0f;
    const uint64_t qlast = (end - 1) >> 2;
    for (uint64_t q0 = (beg >> 2) + lane; q0 <= qlast; q0 += 256) {
        RowLoads<I16> L;
        row_issue<64, I16>(Wd4, idx4, beg, end, q0, L);
        row_consume<64, I16>(L, beg, end, q0, xs, a0, a1, a2, a3);
    }
    return group_sum<64>((a0 + a1) + (a2 + a3));
}

template <int G, typename IdxT>
__device__ __forceinline__ float group_row_dot(const float *__restrict__ Wd, const IdxT *__restrict__ idx,
                                               uint64_t base, uint32_t cnt, const float *xs, uint32_t sub)
{
    float a = 0.0f;
    for (uint32_t j = sub; j < cnt; j += G) a = __builtin_fmaf(Wd[base + j], xs[idx[base + j]], a);
    return group_sum<G>(a);
}

// G lanes per row: a wave works on 64/G rows at a time (whole waves for rows longer than 512
// slots, a half, a quarter or an eighth of a wave for shorter ones, so that short rows do not leave lanes idle).
template <bool XLDS, int G, bool I16>
__global__ __launch_bounds__(kBlock)
void matvec_rows_kernel(const float *__restrict__ Wd, const void *__restrict__ idx,
                        const uint32_t *__restrict__ nnz, uint32_t count, uint32_t r,
                        const float *__restrict__ x, uint32_t n,
                        const float *__restrict__ bias, float *__restrict__ y)
{
    extern __shared__ float lds_x[];
    constexpr uint32_t RPW = 64 / G;                                     // rows per wave
    const uint32_t lane = threadIdx.x & 63u, sub = lane % G, grp = lane / G;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6));
    const uint32_t stride = gridDim.x * kWavesPerBlock * RPW;            // rows between a group's consecutive rows
    const f32x4 *Wd4 = reinterpret_cast<const f32x4 *>(Wd);
    const typename ColGroup<I16>::T *idx4 = reinterpret_cast<const typename ColGroup<I16>::T *>(idx);
    // Rows are pipelined: the first 16 G slots of the next row are requested before the current
    // row is reduced, and those of the group's first row before x is staged, so that a wave always
    // has a row's worth of loads in flight.  Row lengths are fetched two rows ahead, so that
    // requesting a row never waits for its length.
    uint32_t row = wave * RPW + grp;
    uint64_t beg = (uint64_t)row * r, end = beg + (row < count ? nnz[row] : 0u);
    uint32_t len1 = (uint64_t)row + stride < count ? nnz[row + stride] : 0u;          // length of the next row
    RowLoads<I16> cur, nxt;
    if (row < count) row_issue<G, I16>(Wd4, idx4, beg, end, (beg >> 2) + sub, cur);
    const float *xs = stage_x<XLDS>(x, n, lds_x);
    // all groups of a wave make the same number of trips (the reductions need every lane)
    for (uint32_t base = wave * RPW; base < count; base += stride, row += stride) {
        const uint64_t nrow = (uint64_t)row + stride;
        const uint64_t nbeg = nrow * r, nend = nbeg + len1;
        if (nrow < count) row_issue<G, I16>(Wd4, idx4, nbeg, nend, (nbeg >> 2) + sub, nxt);
        const uint32_t len2 = nrow + stride < count ? nnz[nrow + stride] : 0u;
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        if (row < count && end > beg) {
            const uint64_t qlast = (end - 1) >> 2;
            uint64_t q0 = (beg >> 2) + sub;
            row_consume<G, I16>(cur, beg, end, q0, xs, a0, a1, a2, a3);
            for (q0 += 4 * G; q0 <= qlast; q0 += 4 * G) {        // rows longer than one pass
                RowLoads<I16> more;
                row_issue<G, I16>(Wd4, idx4, beg, end, q0, more);
                row_consume<G, I16>(more, beg, end, q0, xs, a0, a1, a2, a3);
            }
        }
        const float s = group_sum<G>((a0 + a1) + (a2 + a3));
        if (sub == 0 && row < count) y[row] = (bias ? bias[row] : 0.0f) + s;
        cur = nxt;
        beg = nbeg;
        end = nend;
        len1 = len2;
    }
}

// Rows of at most G*T nonzeros, G lanes per row.  Such a row is a chain of memory round trips and
// nothing else, so all of a group's first row is requested before x is staged.
template <bool XLDS, int G, int T, typename IdxT>
__device__ __forceinline__ void short_rows(const float *__restrict__ Wd, const IdxT *__restrict__ idx,
                                           const uint2 *__restrict__ rows, uint32_t count, uint32_t block, uint32_t blocks,
                                           uint32_t r, const float *__restrict__ x, uint32_t n, float *lds_x,
                                           const float *__restrict__ bias, float *__restrict__ y)
{
    const uint32_t sub = threadIdx.x % G;
    const uint32_t stride = blocks * (kBlock / G);
    uint32_t g = block * (kBlock / G) + threadIdx.x / G;
    const uint2 e = g < count ? rows[g] : make_uint2(0u, 0u);
    uint2 en = g + stride < count ? rows[g + stride] : make_uint2(0u, 0u);     // the group's next task, a row ahead
    const uint64_t base = (uint64_t)e.x * r;
    float w[T];
    uint32_t c[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const uint32_t j = sub + G * t;
        w[t] = j < e.y ? Wd[base + j] : 0.0f;
        c[t] = j < e.y ? idx[base + j] : 0u;
    }
    const float *xs = stage_x<XLDS>(x, n, lds_x);
    if (g < count) {
        float a = 0.0f;
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const float xv = sub + G * t < e.y ? xs[c[t]] : 0.0f;      // x may be null when nothing is stored
            a = __builtin_fmaf(w[t], xv, a);
        }
        for (uint32_t j = sub + G * T; j < e.y; j += G) a = __builtin_fmaf(Wd[base + j], xs[idx[base + j]], a);
        a = group_sum<G>(a);
        if (sub == 0) y[e.x] = (bias ? bias[e.x] : 0.0f) + a;
    }
    for (g += stride; g < count; g += stride) {
        const uint2 ec = en;
        if (g + stride < count) en = rows[g + stride];
        const float s = group_row_dot<G>(Wd, idx, (uint64_t)ec.x * r, ec.y, xs, sub);
        if (sub == 0) y[ec.x] = (bias ? bias[ec.x] : 0.0f) + s;
    }
}

struct BinArgs {
    const uint2 *rowswg, *rows64, *rows16, *rows4;   // (row, nonzeros of the row) per length class
    uint32_t nwg, n64, n16, n4;                      // rows per class
    uint32_t bwg, b64, b16;                          // workgroups given to the workgroup-, 64- and 16-lane classes
};

constexpr uint32_t kBinnedTailBytes = 64;            // behind x in LDS: the 16 waves' partial sums of a workgroup-wide row

template <bool XLDS, bool I16>
__global__ __launch_bounds__(kBlock, 8)          // 64 registers: two workgroups per compute unit
void matvec_binned_kernel(const float *__restrict__ Wd, const void *__restrict__ idxv, BinArgs ba, uint32_t r,
                          const float *__restrict__ x, uint32_t n,
                          const float *__restrict__ bias, float *__restrict__ y)
{
    extern __shared__ float lds_x[];
    uint32_t b = blockIdx.x;
    if (b < ba.bwg) {
        // Rows of more than 4096 nonzeros: the 16 waves take the row's passes of 1024 slots in turn,
        // the 16 partial sums meet in LDS (behind x) and are added in wave order.
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const f32x4 *Wd4 = reinterpret_cast<const f32x4 *>(Wd);
        const typename ColGroup<I16>::T *idx4 = reinterpret_cast<const typename ColGroup<I16>::T *>(idxv);
        float *part = lds_x + (XLDS ? ((n + 3u) & ~3u) : 0u);
        const float *xs = stage_x<XLDS>(x, n, lds_x);
        for (uint32_t g = b; g < ba.nwg; g += ba.bwg) {
            const uint2 e = ba.rowswg[g];
            const uint64_t beg = (uint64_t)e.x * r, end = beg + e.y;
            const uint64_t qlast = (end - 1) >> 2;                  // e.y > 4096
            float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
            for (uint64_t q = (beg >> 2) + wave * 256u + lane; q <= qlast; q += 256u * kWavesPerBlock) {
                RowLoads<I16> L;
                row_issue<64, I16>(Wd4, idx4, beg, end, q, L);
                row_consume<64, I16>(L, beg, end, q, xs, a0, a1, a2, a3);
            }
            const float s = group_sum<64>((a0 + a1) + (a2 + a3));
            if (lane == 0) part[wave] = s;
            __syncthreads();
            if (threadIdx.x == 0) {
                float t = part[0];
#pragma unroll
                for (int w = 1; w < kWavesPerBlock; ++w) t += part[w];
                y[e.x] = (bias ? bias[e.x] : 0.0f) + t;
            }
            __syncthreads();                                        // part[] is reused by the next row
        }
        return;
    }
    b -= ba.bwg;
    if (b < ba.b64) {
        // A wave's first row (its only one unless the class has more rows than the launch has waves):
        // where it is and how long comes in one load, issued before x is staged.  The row itself is
        // requested after the staging: asked for earlier, it delays x (loads return to a wave in
        // order) and with it the barrier; measured 1.3 us slower on the Zipf matrix.
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t stride = ba.b64 * kWavesPerBlock;
        const f32x4 *Wd4 = reinterpret_cast<const f32x4 *>(Wd);
        const typename ColGroup<I16>::T *idx4 = reinterpret_cast<const typename ColGroup<I16>::T *>(idxv);
        uint32_t g = __builtin_amdgcn_readfirstlane(b * kWavesPerBlock + (threadIdx.x >> 6));
        const uint2 e = g < ba.n64 ? ba.rows64[g] : make_uint2(0u, 0u);
        // the wave's next task, requested a row ahead so that its row never waits for it
        uint2 en = g + stride < ba.n64 ? ba.rows64[g + stride] : make_uint2(0u, 0u);
        const uint64_t beg = (uint64_t)e.x * r, end = beg + e.y;
        const uint64_t q0 = (beg >> 2) + lane;
        const float *xs = stage_x<XLDS>(x, n, lds_x);
        RowLoads<I16> A;
        if (e.y > 0) row_issue<64, I16>(Wd4, idx4, beg, end, q0, A);
        if (g < ba.n64) {
            float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
            if (e.y > 0) {
                row_consume<64, I16>(A, beg, end, q0, xs, a0, a1, a2, a3);
                const uint64_t qlast = (end - 1) >> 2;
                for (uint64_t q = q0 + 256; q <= qlast; q += 256) {
                    RowLoads<I16> L;
                    row_issue<64, I16>(Wd4, idx4, beg, end, q, L);
                    row_consume<64, I16>(L, beg, end, q, xs, a0, a1, a2, a3);
                }
            }
            const float s = group_sum<64>((a0 + a1) + (a2 + a3));
            if (lane == 0) y[e.x] = (bias ? bias[e.x] : 0.0f) + s;
        }
        for (g += stride; g < ba.n64; g += stride) {
            const uint2 ec = en;
            if (g + stride < ba.n64) en = ba.rows64[g + stride];
            const uint64_t nbeg = (uint64_t)ec.x * r;
            const float s = wave_row_dot<I16>(Wd4, idx4, nbeg, nbeg + ec.y, xs, lane);
            if (lane == 0) y[ec.x] = (bias ? bias[ec.x] : 0.0f) + s;
        }
    } else if (b < ba.b64 + ba.b16) {
        const typename ColGroup<I16>::E *idx = reinterpret_cast<const typename ColGroup<I16>::E *>(idxv);
        short_rows<XLDS, 16, 8>(Wd, idx, ba.rows16, ba.n16, b - ba.b64, ba.b16, r, x, n, lds_x, bias, y);
    } else {
        const typename ColGroup<I16>::E *idx = reinterpret_cast<const typename ColGroup<I16>::E *>(idxv);
        short_rows<XLDS, 4, 4>(Wd, idx, ba.rows4, ba.n4, b - ba.b64 - ba.b16, gridDim.x - ba.bwg - ba.b64 - ba.b16, r, x, n,
                               lds_x, bias, y);
    }
}

template <bool XLDS, typename IdxT>
__global__ __launch_bounds__(kBlock)
void matvec_slot_kernel(const float *__restrict__ WdT, const IdxT *__restrict__ idxT,
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

// LDS staging of x is worth its per-workgroup copy only when a workgroup then
// serves many nonzeros from it; it needs n floats of LDS (set up once per kernel).
template <typename K>
bool use_lds(so_ctx *ctx, K kernel, uint32_t n, uint64_t nnz_total, uint32_t blocks, size_t extra = 0)
{
    const size_t lds = (size_t)n * sizeof(float) + extra;
    if (n == 0 || lds > (size_t)ctx->max_lds_bytes) return false;
    if (nnz_total < (uint64_t)n * blocks) return false;   // fewer gathers than staged elements
    if (lds > 48 * 1024 && so_allow_big_lds(ctx, (const void *)kernel) != hipSuccess) return false;
    return true;
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
        // Length classes for skewed rows (the widest row far above the mean).  For even rows the row kernel, which
        // requests a wave's next row while it sums the current one, is the better one except on 16-bit columns
        // where the length-class launch fills its two workgroups per compute unit with two or three rows per wave
        // (16384 columns, 820 nonzeros per row; rows / us row kernel / us length classes: 8192 / 9.3 / 10.1,
        // 16384 / 15.6 / 15.0, 24576 / 21.7 / 21.7, 32768 / 27.5 / 28.3, 49152 / 39.3 / 42.4, 65536 / 51 / 56).
        const bool skewed = (uint64_t)E->r * E->m > 2 * E->total_nnz + E->m;
        const uint32_t per_wave_x2 = E->m / (16u * (uint32_t)ctx->compute_units);           // rows per wave of 2 x CUs workgroups, doubled
        const bool few_rows = E->d_idx16 != nullptr && ctx->tune.matvec_idx16 != 0 && per_wave_x2 >= 4 && per_wave_x2 < 6;
        if ((E->layouts & SO_LAYOUT_BINS) && (skewed || few_rows)) layout = SO_LAYOUT_BINS;
        else if ((E->layouts & SO_LAYOUT_SLOT) && E->max_nnz <= 64) layout = SO_LAYOUT_SLOT;
        else layout = SO_LAYOUT_ROW;
    }
    SO_REQUIRE(layout == SO_LAYOUT_ROW || layout == SO_LAYOUT_SLOT || layout == SO_LAYOUT_BINS,
               "so_matvec: unknown layout %d", layout);
    SO_REQUIRE((E->layouts & layout) != 0, "so_matvec: layout %d was not uploaded", layout);

    const uint32_t cus = (uint32_t)ctx->compute_units;
    const size_t lds = (size_t)E->n * sizeof(float);
    // the row-major kernels read the 16-bit copy of the columns when the handle has one
    const bool i16 = E->d_idx16 != nullptr && ctx->tune.matvec_idx16 != 0;
    const void *cols = i16 ? (const void *)E->d_idx16 : (const void *)E->d_idx;
    if (layout == SO_LAYOUT_ROW) {
        // Lanes per row by the longest row (one pass of 16 G slots should cover it), but never so
        // few that compute units are left without rows.
        uint32_t G = E->max_nnz <= 128 ? 8u : E->max_nnz <= 256 ? 16u : E->max_nnz <= 512 ? 32u : 64u;
        if (ctx->tune.matvec_lanes) G = (uint32_t)ctx->tune.matvec_lanes;
        else
            while (G < 64 && so_ceil_div(E->m, kWavesPerBlock * (64u / G)) < cus) G *= 2;
        // One resident workgroup per compute unit (the pipelined rows need the registers); each of
        // its 16 waves keeps two passes' loads in flight.
        const uint32_t blocks = std::max(1u, std::min(so_ceil_div(E->m, kWavesPerBlock * (64u / G)), cus));
#define SO_MV_ROWS(G, I16)                                                                                         \
        do {                                                                                                       \
            if (use_lds(ctx, matvec_rows_kernel<true, G, I16>, E->n, E->total_nnz, blocks))                        \
                matvec_rows_kernel<true, G, I16><<<blocks, kBlock, lds, ctx->stream>>>(E->d_Wd, cols, E->d_nnz, E->m, E->r, \
                                                                                       dx, E->n, dBias, dy);       \
            else                                                                                                   \
                matvec_rows_kernel<false, G, I16><<<blocks, kBlock, 0, ctx->stream>>>(E->d_Wd, cols, E->d_nnz, E->m, E->r,  \
                                                                                      dx, E->n, dBias, dy);        \
        } while (0)
#define SO_MV_ROWS_G(I16)                                                                                          \
        do {                                                                                                       \
            if (G == 8) SO_MV_ROWS(8, I16);                                                                        \
            else if (G == 16) SO_MV_ROWS(16, I16);                                                                 \
            else if (G == 32) SO_MV_ROWS(32, I16);                                                                 \
            else SO_MV_ROWS(64, I16);                                                                              \
        } while (0)
        if (i16) SO_MV_ROWS_G(true);
        else SO_MV_ROWS_G(false);
#undef SO_MV_ROWS_G
#undef SO_MV_ROWS
    } else if (layout == SO_LAYOUT_SLOT) {
        const uint32_t blocks = std::max(1u, std::min(so_ceil_div(E->m, kBlock), 2u * cus));
#define SO_MV_SLOT(T, COLS)                                                                                        \
        do {                                                                                                       \
            if (use_lds(ctx, matvec_slot_kernel<true, T>, E->n, E->total_nnz, blocks))                             \
                matvec_slot_kernel<true, T><<<blocks, kBlock, lds, ctx->stream>>>(E->d_WdT, COLS, E->d_nnz, E->m,  \
                                                                                  dx, E->n, dBias, dy);            \
            else                                                                                                   \
                matvec_slot_kernel<false, T><<<blocks, kBlock, 0, ctx->stream>>>(E->d_WdT, COLS, E->d_nnz, E->m,   \
                                                                                 dx, E->n, dBias, dy);             \
        } while (0)
        if (E->d_idxT16 && ctx->tune.matvec_idx16 != 0) SO_MV_SLOT(uint16_t, E->d_idxT16);
        else SO_MV_SLOT(uint32_t, E->d_idxT);
#undef SO_MV_SLOT
    } else {
        // One launch over the four length classes.  bins[] is ordered 4, 16, 64 lanes, workgroup.
        BinArgs ba;
        ba.rowswg = reinterpret_cast<const uint2 *>(E->bins[3].d_rows);  ba.nwg = E->bins[3].count;
        ba.bwg = std::min(ba.nwg, cus);
        ba.rows4 = reinterpret_cast<const uint2 *>(E->bins[0].d_rows);   ba.n4 = E->bins[0].count;
        ba.rows16 = reinterpret_cast<const uint2 *>(E->bins[1].d_rows);  ba.n16 = E->bins[1].count;
        ba.rows64 = reinterpret_cast<const uint2 *>(E->bins[2].d_rows);  ba.n64 = E->bins[2].count;
        ba.b64 = std::min(so_ceil_div(ba.n64, kWavesPerBlock), 2u * cus);
        ba.b16 = std::min(so_ceil_div(ba.n16, kBlock / 16), std::max(1u, cus / 4));
        const uint32_t b4 = std::min(so_ceil_div(ba.n4, kBlock / 4), std::max(1u, cus / 4));
        // Staging x pays while a workgroup gathers at least as many elements as it stages (use_lds): rather than
        // give that up, a launch with few nonzeros per workgroup takes fewer workgroups of the wave-per-row class,
        // down to one per compute unit (8192 rows of 820 nonzeros: 20.8 us unstaged on 512 workgroups).
        if (E->n > 0) {
            const uint64_t pays = E->total_nnz / E->n;                       // workgroups for which staging pays
            const uint32_t others = ba.bwg + ba.b16 + b4;
            if ((uint64_t)others + ba.b64 > pays && ba.b64 > cus)
                ba.b64 = (uint32_t)std::max<uint64_t>(cus, pays > others ? pays - others : 0);
        }
        const uint32_t blocks = ba.bwg + ba.b64 + ba.b16 + b4;
        if (blocks == 0) return SO_OK;
        // x padded to whole 16-byte groups, then the partial sums of a workgroup-wide row
        const size_t lds_tail = (((size_t)E->n + 3) & ~(size_t)3) * sizeof(float) + kBinnedTailBytes;
#define SO_MV_BINNED(I16)                                                                                          \
        do {                                                                                                       \
            if (use_lds(ctx, matvec_binned_kernel<true, I16>, E->n, E->total_nnz, blocks, lds_tail - lds))         \
                matvec_binned_kernel<true, I16><<<blocks, kBlock, lds_tail, ctx->stream>>>(E->d_Wd, cols, ba, E->r, \
                                                                                           dx, E->n, dBias, dy);   \
            else                                                                                                   \
                matvec_binned_kernel<false, I16><<<blocks, kBlock, kBinnedTailBytes, ctx->stream>>>(               \
                    E->d_Wd, cols, ba, E->r, dx, E->n, dBias, dy);                                                 \
        } while (0)
        if (i16) SO_MV_BINNED(true);
        else SO_MV_BINNED(false);
#undef SO_MV_BINNED
    }
    SO_LAUNCH_CHECK();
    return SO_OK;
}
