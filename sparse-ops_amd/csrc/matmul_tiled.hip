// The LDS-staged matmul kernel (SO_LAYOUT_TILED) and its launcher.  It lives in its own file
// because it is compiled with the instruction scheduler's max-ILP strategy (see the Makefile):
// measured 1 % faster for this kernel and 10 % slower for the row kernel's few-wave variant.
#include "so_internal.h"
#include "dpp_steps.h"
#include "lds_sync.h"

namespace {

// ---------------------------------------------------------------------------
// LDS-staged variant (SO_LAYOUT_TILED).
//
// The row kernel above moves every X operand through the vector L1, which
// sustains about 50 bytes/clk per CU; LDS sustains five times that for 16-byte
// reads (255 bytes/clk per CU measured).  Here a workgroup of 16 waves owns 64 rows and one slab of 64 dense
// columns, and streams the slab X[:, c0..c0+64) through LDS in tiles of 256 rows
// (64 KB, double-buffered: the next tile is fetched into registers while the
// current one is consumed; progress counters in LDS, not barriers, tell a wave when
// a buffer may be read or overwritten).  A wave works on a quad of four rows, 16 lanes per
// row, four columns per lane, so one ds_read_b128 per lane serves four FMAs.  The
// (weight, LDS offset) pairs of a quad's rows for the current tile sit in lanes
// (chunk of 16 steps per row, fetched one tile ahead and before the X prefetch,
// so waiting for them never waits for X) and are broadcast inside each 16-lane
// row with DPP row_newbcast.  Each row still receives its nonzeros in ascending
// slot order starting from the bias: results are bit-identical to the row kernel.
// A step that a row of the quad does not have is the pair (-0, zero row):
// fma(-0, 0, acc) leaves acc unchanged, a -0 accumulator included.
// ---------------------------------------------------------------------------

constexpr int kTiledWaves = so_tiled::kWavesPerGroup;
constexpr int kMaxChunks = 3;   // chunks of 16 steps held in registers per tile; more run from memory

template <int ACT>
__global__ __launch_bounds__(kTiledWaves * 64)
void ellpack_matmul_tiled_kernel(const so_tile_entry *__restrict__ entries, const so_tile_info *__restrict__ info,
                                 const uint32_t *__restrict__ quad_rows, uint32_t nquads, uint32_t ntiles,
                                 uint32_t n, const float *__restrict__ X, uint32_t C,
                                 const float *__restrict__ bias, float *__restrict__ Y,
                                 uint32_t nslabs, uint32_t ngroups, bool group_major, so_lds::wait_status ws)
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
    // Progress counters instead of a barrier per tile (lds_sync.h): [0], [1] tiles stored into buffer
    // 0 / 1 (x 16 waves), [2], [3] tiles read out of them.  Measured on the 4096 x 4096 @ 90 % x 256
    // launch: 39.7 -> 37.8 us (storing after the second chunk instead of the first: 43.4).
    static_assert(so_tiled::kSyncOff + so_lds::kSyncBytes <= so_tiled::kLdsBytes, "room for the counters");
    const uint32_t sync_base = so_lds::lds_address(lds + so_tiled::kSyncOff);
    if (tid < 4) reinterpret_cast<uint32_t *>(lds + so_tiled::kSyncOff)[tid] = tid == 0 ? 16u : 0u;
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
        const bool more = t + 1 < ntiles;
#pragma unroll
        for (int c = 0; c < kMaxChunks; ++c) {
            if (c == 1 && more) {
                // the wave's part of the next tile, once every wave has finished the tile before this one
                so_lds::wait(sync_base + 8u + ((t + 1u) & 1u) * 4u, 16u * ((t + 1u) / 2u), ws);
                lstore((t + 1) & 1u);
                so_lds::signal(sync_base + ((t + 1u) & 1u) * 4u, lane);
            }
            if (cur.steps > 16u * c) so_dpp::tiled_chunk(base, ew[c], eo[c], cur.steps - 16u * c, acc);
        }
        for (uint32_t c = kMaxChunks; c * 16u < cur.steps; ++c) {
            const so_tile_entry e = lane_ent[(size_t)(cur.chunk0 + c) * 64];
            so_dpp::tiled_chunk(base, e.w, e.off, cur.steps - 16u * c, acc);
        }
        so_lds::signal(sync_base + 8u + (t & 1u) * 4u, lane);                                     // done reading this tile's buffer
        if (more) so_lds::wait(sync_base + ((t + 1u) & 1u) * 4u, 16u * ((t + 1u) / 2u + 1u), ws);     // the next tile is complete
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
        T.d_entries, T.d_info, T.d_rows, T.nquads, T.ntiles, E->n, dX, C, dBias, dY, nslabs, ngroups, grpmajor,
        so_lds::wait_status{ctx->tune.wait_spins >= 0 ? (uint32_t)ctx->tune.wait_spins : so_lds::kSyncSpins, ctx->d_wait_gave_up});
    ctx->waits_pending = true;
    return SO_OK;
}

} // namespace

so_status so_matmul_tiled_launch(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                                 const float *dBias, float *dY, int act)
{
    switch (act) {
    case SO_ACT_RELU:    return launch_tiled<SO_ACT_RELU>(ctx, E, dX, C, dBias, dY);
    case SO_ACT_SIGMOID: return launch_tiled<SO_ACT_SIGMOID>(ctx, E, dX, C, dBias, dY);
    case SO_ACT_TANH:    return launch_tiled<SO_ACT_TANH>(ctx, E, dX, C, dBias, dY);
    default:             return launch_tiled<SO_ACT_NONE>(ctx, E, dX, C, dBias, dY);
    }
}
