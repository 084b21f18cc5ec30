// so_matmul: Y[m x C] = act(E * X[n x C] + bias) on gfx950.
//
// One wavefront owns one ELLPACK row and one tile of 64*VEC dense columns.  The
// row's weights and column indices are wave-uniform, so they are fetched with
// scalar loads into SGPRs; every gathered X row segment X[j, c0 .. c0+64*VEC) is
// one fully coalesced vector load; each lane keeps VEC fp32 accumulators that
// start at bias[i] and receive one fused multiply-add per stored nonzero in
// ascending slot order -- the rounding sequence of the reference's inner loop
// (src/ellpack_matmul.cpp:51-66) -- followed by the fused epilogue.
//
// Workgroups are numbered so that each of the 8 XCDs (workgroup id modulo 8)
// works on as few column tiles as possible: an XCD's L2 then has to hold only
// its own tiles' slice of X.
#include "so_internal.h"

#include <cstdlib>

namespace {

constexpr int kWavesPerGroup = 4;

template <int VEC> struct VecT;
template <> struct VecT<1> { using type = float; };
template <> struct VecT<2> { using type = float2; };
template <> struct VecT<4> { using type = float4; };

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&v)[VEC])
{
    using T = typename VecT<VEC>::type;
    const T t = *reinterpret_cast<const T *>(p);
    if constexpr (VEC == 1) { v[0] = t; }
    if constexpr (VEC == 2) { v[0] = t.x; v[1] = t.y; }
    if constexpr (VEC == 4) { v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
}

template <int VEC>
__device__ __forceinline__ void store_vec(float *p, const float (&v)[VEC])
{
    using T = typename VecT<VEC>::type;
    T t;
    if constexpr (VEC == 1) { t = v[0]; }
    if constexpr (VEC == 2) { t.x = v[0]; t.y = v[1]; }
    if constexpr (VEC == 4) { t.x = v[0]; t.y = v[1]; t.z = v[2]; t.w = v[3]; }
    *reinterpret_cast<T *>(p) = t;
}

struct TileMap {
    uint32_t ntiles;      // column tiles
    uint32_t nrowgroups;  // groups of kWavesPerGroup rows
    uint32_t mode;        // 0 plain, 1: ntiles divides 8, 2: 8 divides ntiles
};

// Workgroup id -> (column tile, row group).  XCD = id % 8.
__device__ __forceinline__ bool map_tile(const TileMap tm, uint32_t wg, uint32_t &tile, uint32_t &rg)
{
    const uint32_t xcd = wg & 7u, q = wg >> 3;
    if (tm.mode == 1) {
        const uint32_t per = 8u / tm.ntiles;  // XCDs sharing one tile
        tile = xcd % tm.ntiles;
        rg = xcd / tm.ntiles + per * q;
    } else if (tm.mode == 2) {
        const uint32_t per = tm.ntiles >> 3;  // tiles per XCD
        tile = xcd + 8u * (q % per);
        rg = q / per;
    } else {
        tile = wg % tm.ntiles;
        rg = wg / tm.ntiles;
    }
    return rg < tm.nrowgroups;
}

// FULL: every column tile is complete (C % (64*VEC) == 0), no lane predicate.
// kUnroll: gathers per register batch (two batches are in flight).  8 when the
// chip is full of waves; 32 for launches with only a few waves, where a wave's own
// memory latency is all there is to hide.
template <int VEC, int ACT, bool FULL, int kUnroll>
__global__ __launch_bounds__(kWavesPerGroup * 64)
void ellpack_matmul_kernel(const float *__restrict__ Wd, const uint32_t *__restrict__ idx,
                           const uint32_t *__restrict__ nnz, uint32_t m, uint32_t r,
                           const float *__restrict__ X, uint32_t C,
                           const float *__restrict__ bias, float *__restrict__ Y, TileMap tm)
{
    uint32_t tile, rg;
    if (!map_tile(tm, blockIdx.x, tile, rg)) return;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = __builtin_amdgcn_readfirstlane(rg * kWavesPerGroup + (threadIdx.x >> 6));
    if (row >= m) return;

    const uint32_t col = tile * (64u * VEC) + lane * VEC;
    // A partial tile only happens with VEC == 1 (the host picks VEC so that C % VEC == 0).
    const bool live = FULL || col < C;
    const uint32_t cnt = nnz[row];
    const float *__restrict__ wrow = Wd + (size_t)row * r;
    const uint32_t *__restrict__ irow = idx + (size_t)row * r;
    const float *__restrict__ xcol = X + (live ? col : 0u);

    float acc[VEC];
    const float b = bias ? bias[row] : 0.0f;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = b;

    // Batches of kUnroll nonzeros, double-buffered in registers: the gathers of
    // batch b+1 are issued before batch b is consumed, so a wave always has one
    // batch of loads in flight while it waits for scalar loads or does FMAs.
    // The FMAs themselves stay strictly in slot order.
    float wa[kUnroll], wb[kUnroll];
    float xa[kUnroll][VEC], xb[kUnroll][VEC];
    auto issue = [&](uint32_t j0, float (&w)[kUnroll], float (&x)[kUnroll][VEC]) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            w[u] = wrow[j0 + u];
            load_vec<VEC>(xcol + (size_t)irow[j0 + u] * C, x[u]);
        }
    };
    auto consume = [&](const float (&w)[kUnroll], const float (&x)[kUnroll][VEC]) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(w[u], x[u][v], acc[v]);
    };
    const uint32_t nb = cnt / kUnroll;
    if (nb) issue(0, wa, xa);
    uint32_t bi = 0;
    for (; bi + 1 < nb; bi += 2) {
        issue((bi + 1) * kUnroll, wb, xb);
        consume(wa, xa);
        if (bi + 2 < nb) issue((bi + 2) * kUnroll, wa, xa);
        consume(wb, xb);
    }
    if (nb & 1u) consume(wa, xa);
    // The last, partial batch.  With few waves on the chip (kUnroll 32) all its gathers are issued at
    // once (slots past the row's end re-read the row's last nonzero) and the multiply-adds run under
    // a wave-uniform test per slot: one memory round trip instead of one per nonzero.  With the chip
    // full of waves the plain loop is faster (no redundant gathers; other waves hide the latency).
    if constexpr (kUnroll >= 32) {
        if (const uint32_t rem = cnt - nb * kUnroll) {
            const uint32_t j0 = nb * kUnroll;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const uint32_t j = j0 + min((uint32_t)u, rem - 1u);
                wa[u] = wrow[j];
                load_vec<VEC>(xcol + (size_t)irow[j] * C, xa[u]);
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                if ((uint32_t)u < rem) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(wa[u], xa[u][v], acc[v]);
                }
        }
    } else {
        for (uint32_t j = nb * kUnroll; j < cnt; ++j) {
            const float w = wrow[j];
            float x[VEC];
            load_vec<VEC>(xcol + (size_t)irow[j] * C, x);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(w, x[v], acc[v]);
        }
    }

    if (live) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = so_epilogue<ACT>(acc[v]);
        store_vec<VEC>(Y + (size_t)row * C + col, acc);
    }
}

template <int VEC, int ACT, int UNROLL = 8>
void launch(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C, const float *dBias, float *dY)
{
    TileMap tm;
    tm.ntiles = so_ceil_div(C, 64u * VEC);
    tm.nrowgroups = so_ceil_div(E->m, kWavesPerGroup);
    tm.mode = (tm.ntiles <= 8 && 8 % tm.ntiles == 0) ? 1 : (tm.ntiles % 8 == 0 ? 2 : 0);
    uint32_t blocks;
    if (tm.mode == 1) blocks = so_ceil_div(tm.nrowgroups, 8u / tm.ntiles) * 8u;
    else blocks = tm.ntiles * tm.nrowgroups;
    const bool full = C % (64u * VEC) == 0;
    auto k = full ? ellpack_matmul_kernel<VEC, ACT, true, UNROLL> : ellpack_matmul_kernel<VEC, ACT, false, UNROLL>;
    k<<<blocks, kWavesPerGroup * 64, 0, ctx->stream>>>(E->d_Wd, E->d_idx, E->d_nnz, E->m, E->r,
                                                       dX, C, dBias, dY, tm);
}

template <int VEC, int UNROLL = 8>
void launch_act(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C, const float *dBias,
                float *dY, int act)
{
    switch (act) {
    case SO_ACT_RELU:    launch<VEC, SO_ACT_RELU, UNROLL>(ctx, E, dX, C, dBias, dY); break;
    case SO_ACT_SIGMOID: launch<VEC, SO_ACT_SIGMOID, UNROLL>(ctx, E, dX, C, dBias, dY); break;
    case SO_ACT_TANH:    launch<VEC, SO_ACT_TANH, UNROLL>(ctx, E, dX, C, dBias, dY); break;
    default:             launch<VEC, SO_ACT_NONE, UNROLL>(ctx, E, dX, C, dBias, dY); break;
    }
}

// ---------------------------------------------------------------------------
// Few rows (a classifier head): rows x column tiles give fewer waves than the chip
// has CUs, so a wave's own gather latency is all there is to hide, and the bytes it
// can keep in flight are bounded by its registers.  Here a workgroup of 16 waves
// shares one (row, 64-column tile): the waves split the row's nonzeros among them
// for the gathers (16 times the loads in flight), park the gathered X segments in
// LDS, and the first wave then runs the multiply-adds over them in slot order
// starting from the bias -- the same rounding sequence as the row kernel.
// ---------------------------------------------------------------------------

constexpr int kShareWaves = 16;
constexpr int kSharePerWave = 32;                           // gathers per wave and chunk
constexpr int kShareChunk = kShareWaves * kSharePerWave;    // slots per chunk: 128 KB of X segments
constexpr size_t kShareLdsBytes = (size_t)kShareChunk * 64 * sizeof(float) + kShareChunk * sizeof(float);

template <int ACT>
__global__ __launch_bounds__(kShareWaves * 64)
void ellpack_matmul_shared_gather_kernel(const float *__restrict__ Wd, const uint32_t *__restrict__ idx,
                                         const uint32_t *__restrict__ nnz, uint32_t r,
                                         const float *__restrict__ X, uint32_t C,
                                         const float *__restrict__ bias, float *__restrict__ Y, uint32_t ntiles)
{
    extern __shared__ __attribute__((aligned(16))) float share_lds[];
    float4 *xs4 = reinterpret_cast<float4 *>(share_lds);   // [kShareChunk / 4][64 lanes][4 slots]
    float *ws = share_lds + (size_t)kShareChunk * 64;      // [kShareChunk]
    const uint32_t tile = blockIdx.x % ntiles, row = blockIdx.x / ntiles;   // the grid is exactly m * ntiles
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t col = tile * 64u + lane;
    const bool live = col < C;
    const uint32_t cnt = nnz[row];
    const float *__restrict__ wrow = Wd + (size_t)row * r;
    const uint32_t *__restrict__ irow = idx + (size_t)row * r;
    const float *__restrict__ xcol = X + (live ? col : 0u);
    float acc = bias ? bias[row] : 0.0f;

    for (uint32_t s0 = 0; s0 < cnt; s0 += kShareChunk) {
        const uint32_t chunk = min((uint32_t)kShareChunk, cnt - s0);
        const uint32_t w0 = wave * kSharePerWave;        // this wave gathers slots s0 + w0 .. + kSharePerWave
        if (w0 < chunk) {
            const uint32_t mine = min((uint32_t)kSharePerWave, chunk - w0);
            float x[kSharePerWave];
#pragma unroll
            for (int u = 0; u < kSharePerWave; ++u) {    // slots past the wave's share re-read its last one
                const uint32_t j = s0 + w0 + min((uint32_t)u, mine - 1u);
                x[u] = xcol[(size_t)irow[j] * C];
            }
            if (lane < mine) ws[w0 + lane] = wrow[s0 + w0 + lane];
            // four consecutive slots of a lane side by side: the wave that multiplies takes them with one read
#pragma unroll
            for (int u = 0; u < kSharePerWave; u += 4)
                if ((uint32_t)u < mine) xs4[((w0 + u) / 4u) * 64u + lane] = make_float4(x[u], x[u + 1], x[u + 2], x[u + 3]);
        }
        __syncthreads();
        if (wave == 0) {
            // One wave, one instruction at a time: what counts is instructions per slot -- a 16-byte read of four
            // weights (every lane the same address), one of this lane's four operands, four multiply-adds.
            uint32_t s = 0;
            for (; s + 8 <= chunk; s += 8) {
                const float4 wa = *reinterpret_cast<const float4 *>(ws + s), wb = *reinterpret_cast<const float4 *>(ws + s + 4);
                const float4 xa = xs4[(s / 4u) * 64u + lane], xb = xs4[(s / 4u + 1u) * 64u + lane];
                acc = __builtin_fmaf(wa.x, xa.x, acc); acc = __builtin_fmaf(wa.y, xa.y, acc);
                acc = __builtin_fmaf(wa.z, xa.z, acc); acc = __builtin_fmaf(wa.w, xa.w, acc);
                acc = __builtin_fmaf(wb.x, xb.x, acc); acc = __builtin_fmaf(wb.y, xb.y, acc);
                acc = __builtin_fmaf(wb.z, xb.z, acc); acc = __builtin_fmaf(wb.w, xb.w, acc);
            }
            for (; s < chunk; ++s) acc = __builtin_fmaf(ws[s], share_lds[(s / 4u) * 256u + lane * 4u + (s & 3u)], acc);
        }
        __syncthreads();                                  // the next chunk overwrites what wave 0 was reading
    }
    if (wave == 0 && live) Y[(size_t)row * C + col] = so_epilogue<ACT>(acc);
}

template <int ACT>
so_status launch_shared_gather(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C, const float *dBias, float *dY)
{
    SO_HIP(so_allow_big_lds(ctx, (const void *)ellpack_matmul_shared_gather_kernel<ACT>));
    const uint32_t ntiles = so_ceil_div(C, 64u);
    ellpack_matmul_shared_gather_kernel<ACT><<<E->m * ntiles, kShareWaves * 64, kShareLdsBytes, ctx->stream>>>(
        E->d_Wd, E->d_idx, E->d_nnz, E->r, dX, C, dBias, dY, ntiles);
    return SO_OK;
}

} // namespace

extern "C" so_status so_matmul_reserve(so_ctx *ctx, const so_ellpack *E, uint32_t C)
{
    SO_REQUIRE(ctx && E, "so_matmul_reserve: null argument");
    if (E->m == 0 || C == 0 || !so_matmul_rbm_applies(ctx, E, C)) return SO_OK;
    const so_status st = so_matmul_rbm_reserve(ctx, E, C);
    return st != SO_OK ? st : so_matmul_rbm_set_pitch(ctx, E, C);
}

extern "C" so_status so_matmul(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                               const float *dBias, float *dY, int act)
{
    SO_REQUIRE(ctx && E, "so_matmul: null argument");
    SO_REQUIRE(act >= SO_ACT_NONE && act <= SO_ACT_TANH, "so_matmul: unknown activation %d", act);
    if (E->m == 0 || C == 0) return SO_OK;  // empty output: nothing to launch
    SO_REQUIRE(dY != nullptr, "so_matmul: Y is null");
    SO_REQUIRE(dX != nullptr || E->total_nnz == 0, "so_matmul: X is null");
    // one workgroup per (4 rows, 64 columns) at most: the grid must fit 31 bits
    SO_REQUIRE(((uint64_t)E->m / 4 + 8) * ((uint64_t)C / 64 + 1) < (1ull << 31), "so_matmul: %u x %u output is too large for one launch", E->m, C);

    // The row-block-merged kernel, on handles uploaded with its layout (accurate to fp32 round-off, not
    // bit-identical to the row order: the caller asked for it by asking for the layout).  It takes one
    // workgroup per (128 rows, 64 columns, share of the columns), so like the LDS-staged kernel it pays
    // when that grid covers most of the chip (SPARSEOPS_MATMUL_RBM=1 forces it, =0 forbids it).
    if (so_matmul_rbm_applies(ctx, E, C) && dX != nullptr && (((uintptr_t)dX | (uintptr_t)dY) & 3) == 0) {
        const uint64_t groups = (uint64_t)E->rbmm.nb * so_ceil_div(C, 64) * E->rbmm.ksplit;
        bool rbm = 4 * groups >= 3 * (uint64_t)ctx->compute_units;
        if (ctx->tune.matmul_rbm >= 0) rbm = ctx->tune.matmul_rbm == 1;
        if (rbm) {
            const so_status st = so_matmul_rbm_launch(ctx, E, dX, C, dBias, dY, act);
            if (st != SO_OK) return st;
            SO_LAUNCH_CHECK();
            return SO_OK;
        }
    }

    const uintptr_t align = (uintptr_t)dX | (uintptr_t)dY;
    // The LDS-staged kernel needs whole float4 column groups.  It takes one
    // workgroup per (64 rows, 64 columns), one workgroup per CU at a time, so it pays
    // only when that grid covers most of the chip; smaller problems stay on the row
    // kernel (SPARSEOPS_MATMUL_TILED=1 forces it, =0 forbids it: tuning and tests).
    bool tiled = (E->layouts & SO_LAYOUT_TILED) && C % 4 == 0 && C >= 16 && (align & 15) == 0 &&
                 (size_t)ctx->max_lds_bytes >= so_tiled::kLdsBytes;
    if (tiled) {
        const uint64_t groups = (uint64_t)so_ceil_div(C, so_tiled::kSlabCols) * so_ceil_div(E->tiled.nquads, so_tiled::kWavesPerGroup);
        if (ctx->tune.matmul_tiled >= 0) tiled = ctx->tune.matmul_tiled == 1;
        else tiled = 4 * groups >= 3 * (uint64_t)ctx->compute_units;
    }
    if (tiled) {
        const so_status st = so_matmul_tiled_launch(ctx, E, dX, C, dBias, dY, act);
        if (st != SO_OK) return st;
        SO_LAUNCH_CHECK();
        return SO_OK;
    }

    // Columns per lane: as wide as alignment allows while every tile stays whole.
    int vec = 1;
    if (C % 256 == 0 && (align & 15) == 0) vec = 4;
    else if (C % 128 == 0 && (align & 7) == 0) vec = 2;
    if ((ctx->tune.matmul_vec == 1 || ctx->tune.matmul_vec == 2) && ctx->tune.matmul_vec < vec) vec = ctx->tune.matmul_vec;   // narrower lanes only
    // Few waves in total (at most one per SIMD even with one column per lane): the
    // launch is latency-bound, so spread it over as many waves as possible and give
    // each wave 2 x 32 gathers in flight.
    const uint64_t row_tiles = (uint64_t)E->m * so_ceil_div(C, 64);
    // At most one (row, tile) per CU and rows long enough to be worth sharing: 16 waves gather for each.
    bool share = row_tiles <= (uint64_t)ctx->compute_units && E->max_nnz >= 128 && (size_t)ctx->max_lds_bytes >= kShareLdsBytes;
    if (ctx->tune.matmul_share >= 0) share = share && ctx->tune.matmul_share == 1;
    if (share) {
        so_status st;
        switch (act) {
        case SO_ACT_RELU:    st = launch_shared_gather<SO_ACT_RELU>(ctx, E, dX, C, dBias, dY); break;
        case SO_ACT_SIGMOID: st = launch_shared_gather<SO_ACT_SIGMOID>(ctx, E, dX, C, dBias, dY); break;
        case SO_ACT_TANH:    st = launch_shared_gather<SO_ACT_TANH>(ctx, E, dX, C, dBias, dY); break;
        default:             st = launch_shared_gather<SO_ACT_NONE>(ctx, E, dX, C, dBias, dY); break;
        }
        if (st != SO_OK) return st;
        SO_LAUNCH_CHECK();
        return SO_OK;
    }
    if (row_tiles <= 4ull * (uint64_t)ctx->compute_units && E->max_nnz >= 64)
        launch_act<1, 32>(ctx, E, dX, C, dBias, dY, act);
    else if (vec == 4) launch_act<4>(ctx, E, dX, C, dBias, dY, act);
    else if (vec == 2) launch_act<2>(ctx, E, dX, C, dBias, dY, act);
    else launch_act<1>(ctx, E, dX, C, dBias, dY, act);
    SO_LAUNCH_CHECK();
    return SO_OK;
}
