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
#include "dpp_steps.h"

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
// LDS in slot order, and the first wave then runs the multiply-adds over them in
// slot order starting from the bias -- the same rounding sequence as the row kernel.
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
    float *xs = share_lds;                              // [kShareChunk][64]
    float *ws = share_lds + (size_t)kShareChunk * 64;   // [kShareChunk]
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
#pragma unroll
            for (int u = 0; u < kSharePerWave; ++u)
                if ((uint32_t)u < mine) xs[(w0 + u) * 64u + lane] = x[u];
        }
        __syncthreads();
        if (wave == 0) {
            uint32_t s = 0;
            for (; s + 8 <= chunk; s += 8) {
                float w[8], x[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) { w[u] = ws[s + u]; x[u] = xs[(s + u) * 64u + lane]; }
#pragma unroll
                for (int u = 0; u < 8; ++u) acc = __builtin_fmaf(w[u], x[u], acc);
            }
            for (; s < chunk; ++s) acc = __builtin_fmaf(ws[s], xs[s * 64u + lane], acc);
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

// ---------------------------------------------------------------------------
// LDS-staged variant (SO_LAYOUT_TILED).
//
// The row kernel above moves every X operand through the vector L1, which
// sustains about 50 bytes/clk per CU; LDS sustains three times that for 16-byte
// reads.  Here a workgroup of 16 waves owns 64 rows and one slab of 64 dense
// columns, and streams the slab X[:, c0..c0+64) through LDS in tiles of 256 rows
// (64 KB, double-buffered: the next tile is fetched into registers while the
// current one is consumed).  A wave works on a quad of four rows, 16 lanes per
// row, four columns per lane, so one ds_read_b128 per lane serves four FMAs.  The
// (weight, LDS offset) pairs of a quad's rows for the current tile sit in lanes
// (chunk of 16 steps per row, fetched one tile ahead and before the X prefetch,
// so waiting for them never waits for X) and are broadcast inside each 16-lane
// row with DPP row_newbcast.  Each row still receives its nonzeros in ascending
// slot order starting from the bias: results are bit-identical to the row kernel.
// A step that a row of the quad does not have is the pair (0, zero row):
// fma(0, 0, acc) leaves acc unchanged.
// ---------------------------------------------------------------------------

constexpr int kTiledWaves = 16;
constexpr int kMaxChunks = 3;   // chunks of 16 steps held in registers per tile; more run from memory

template <int ACT>
__global__ __launch_bounds__(kTiledWaves * 64)
void ellpack_matmul_tiled_kernel(const so_tile_entry *__restrict__ entries, const so_tile_info *__restrict__ info,
                                 const uint32_t *__restrict__ quad_rows, uint32_t nquads, uint32_t ntiles,
                                 uint32_t n, const float *__restrict__ X, uint32_t C,
                                 const float *__restrict__ bias, float *__restrict__ Y,
                                 uint32_t nslabs, uint32_t ngroups, bool group_major)
{
    constexpr uint32_t KT = so_tiled::kTileRows, ROWB = so_tiled::kSlabCols * 4, TILE = so_tiled::kTileBytes;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    // Workgroup id -> (column slab, group of 16 quads).  Workgroup ids go round the 8 XCDs, each
    // with its own L2.  group_major: an XCD takes whole groups, the slabs of a group one after the
    // other, so the group's entries come from HBM once and from that L2 for the other slabs
    // (chosen when all of X fits an L2).  Otherwise an XCD keeps to one slab when the slab count
    // divides 8, so that its L2 has to hold a single slab of X.
    uint32_t slab, grp;
    {
        const uint32_t xcd = blockIdx.x & 7u, q = blockIdx.x >> 3;
        if (group_major) { slab = q % nslabs; grp = (q / nslabs) * 8u + xcd; }
        else if (8 % nslabs == 0) { slab = xcd % nslabs; grp = xcd / nslabs + (8 / nslabs) * q; }
        else { slab = blockIdx.x % nslabs; grp = blockIdx.x / nslabs; }
        if (grp >= ngroups) return;
    }
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t g = lane >> 4, cq = lane & 15u;
    const uint32_t quad = grp * kTiledWaves + wave;
    const bool quad_ok = quad < nquads;
    const uint32_t row = quad_ok ? quad_rows[(size_t)quad * 4 + g] : 0xffffffffu;
    const uint32_t c0 = slab * so_tiled::kSlabCols;
    const uint32_t col = c0 + cq * 4;

    float acc[4];
    {
        const float b = (bias && row != 0xffffffffu) ? bias[row] : 0.0f;
        acc[0] = acc[1] = acc[2] = acc[3] = b;
    }

    // Tile loader: thread -> X row (tid >> 4) + 64*i of the tile, column quad tid & 15.
    const uint32_t lr = tid >> 4, lc = tid & 15u;
    const bool lcol_ok = c0 + lc * 4 < C;            // C is a multiple of 4
    const float *xsrc = X + (size_t)lr * C + c0 + lc * 4;
    float4 pre[4];
    const bool slab_full = c0 + so_tiled::kSlabCols <= C;       // wave-uniform
    auto gload = [&](uint32_t t) {
        if (slab_full && (t + 1) * KT <= n) {                    // whole tile inside X: no per-lane tests
#pragma unroll
            for (int i = 0; i < 4; ++i)
                pre[i] = *reinterpret_cast<const float4 *>(xsrc + (size_t)(t * KT + 64 * i) * C);
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t xr = t * KT + lr + 64 * i;
            pre[i] = (lcol_ok && xr < n) ? *reinterpret_cast<const float4 *>(xsrc + (size_t)(t * KT + 64 * i) * C)
                                         : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    auto lstore = [&](uint32_t buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<float4 *>(lds + buf * TILE + (lr + 64 * i) * ROWB + lc * 16) = pre[i];
    };

    const so_tile_info *qi = info + (size_t)(quad_ok ? quad : 0) * ntiles;
    const so_tile_entry *lane_ent = entries + lane;
    float ew[kMaxChunks], nw[kMaxChunks];
    uint32_t eo[kMaxChunks], no[kMaxChunks];
    auto eload = [&](so_tile_info ti, float (&w)[kMaxChunks], uint32_t (&o)[kMaxChunks]) {
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c) {   // unconditional: the array ends with kMaxChunks spare chunks
            const so_tile_entry e = lane_ent[(size_t)(ti.chunk0 + c) * 64];
            w[c] = e.w;
            o[c] = e.off;
        }
    };

    so_tile_info cur = qi[0];
    if (!quad_ok) cur.steps = 0;
    eload(cur, ew, eo);
    if (tid < 16) *reinterpret_cast<float4 *>(lds + so_tiled::kZeroRowOff + tid * 16) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    gload(0);
    lstore(0);
    __syncthreads();

    const uint32_t lane_off = cq * 16;
    for (uint32_t t = 0; t < ntiles; ++t) {
        so_tile_info nxt{0, 0};
        if (t + 1 < ntiles) {
            nxt = qi[t + 1];
            if (!quad_ok) nxt.steps = 0;
            eload(nxt, nw, no);
            gload(t + 1);
        }
        const char *base = lds + (t & 1u) * TILE + lane_off;
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c)
            if (cur.steps > 16u * c) so_dpp::tiled_chunk(base, ew[c], eo[c], cur.steps - 16u * c, acc);
        for (uint32_t c = kMaxChunks; c * 16u < cur.steps; ++c) {
            const so_tile_entry e = lane_ent[(size_t)(cur.chunk0 + c) * 64];
            so_dpp::tiled_chunk(base, e.w, e.off, cur.steps - 16u * c, acc);
        }
        if (t + 1 < ntiles) lstore((t + 1) & 1u);
        __syncthreads();
        cur = nxt;
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c) { ew[c] = nw[c]; eo[c] = no[c]; }
    }
    if (row != 0xffffffffu && col < C) {
        float4 out;
        out.x = so_epilogue<ACT>(acc[0]);
        out.y = so_epilogue<ACT>(acc[1]);
        out.z = so_epilogue<ACT>(acc[2]);
        out.w = so_epilogue<ACT>(acc[3]);
        *reinterpret_cast<float4 *>(Y + (size_t)row * C + col) = out;
    }
}

template <int ACT>
so_status launch_tiled(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C, const float *dBias, float *dY)
{
    const so_tiled &T = E->tiled;
    SO_HIP(so_allow_big_lds(ctx, (const void *)ellpack_matmul_tiled_kernel<ACT>));
    const uint32_t nslabs = so_ceil_div(C, so_tiled::kSlabCols);
    const uint32_t ngroups = so_ceil_div(T.nquads, kTiledWaves);
    // all of X inside one XCD's L2 (4 MB): share a group's entries between its slabs instead of a slab between groups
    const bool grpmajor = (uint64_t)E->n * C * sizeof(float) <= (4ull << 20);
    const uint32_t blocks = grpmajor ? so_ceil_div(ngroups, 8) * 8 * nslabs
                                     : (8 % nslabs == 0) ? so_ceil_div(ngroups, 8 / nslabs) * 8 : nslabs * ngroups;
    ellpack_matmul_tiled_kernel<ACT><<<blocks, kTiledWaves * 64, so_tiled::kLdsBytes, ctx->stream>>>(
        T.d_entries, T.d_info, T.d_rows, T.nquads, T.ntiles, E->n, dX, C, dBias, dY, nslabs, ngroups, grpmajor);
    return SO_OK;
}

} // namespace

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

    const uintptr_t align = (uintptr_t)dX | (uintptr_t)dY;
    // The LDS-staged kernel needs whole float4 column groups.  It takes one
    // workgroup per (64 rows, 64 columns), one workgroup per CU at a time, so it pays
    // only when that grid covers most of the chip; smaller problems stay on the row
    // kernel (SPARSEOPS_MATMUL_TILED=1 forces it, =0 forbids it: tuning and tests).
    bool tiled = (E->layouts & SO_LAYOUT_TILED) && C % 4 == 0 && C >= 16 && (align & 15) == 0 &&
                 (size_t)ctx->max_lds_bytes >= so_tiled::kLdsBytes;
    if (tiled) {
        const uint64_t groups = (uint64_t)so_ceil_div(C, so_tiled::kSlabCols) * so_ceil_div(E->tiled.nquads, kTiledWaves);
        if (ctx->tune.matmul_tiled >= 0) tiled = ctx->tune.matmul_tiled == 1;
        else tiled = 4 * groups >= 3 * (uint64_t)ctx->compute_units;
    }
    if (tiled) {
        so_status st;
        switch (act) {
        case SO_ACT_RELU:    st = launch_tiled<SO_ACT_RELU>(ctx, E, dX, C, dBias, dY); break;
        case SO_ACT_SIGMOID: st = launch_tiled<SO_ACT_SIGMOID>(ctx, E, dX, C, dBias, dY); break;
        case SO_ACT_TANH:    st = launch_tiled<SO_ACT_TANH>(ctx, E, dX, C, dBias, dY); break;
        default:             st = launch_tiled<SO_ACT_NONE>(ctx, E, dX, C, dBias, dY); break;
        }
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
