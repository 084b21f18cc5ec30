// Row-block-merged (RBM) sparse convolution: the reference's blocked-CSC re-encoding of the
// ELLPACK weights (include/rbm_conv.hpp:8-27, src/layers/rbm_conv.cpp:7-73) and the kernel that
// walks it (conv2d_rbm_fmajor_implicit, src/layers/conv_kernels.cpp:66-147), on gfx950.
//
// A block is up to 8 consecutive output channels.  Its union columns -- the (cin, kh, kw) taps
// that at least one channel of the block uses -- are walked once, in ascending order, and the
// input operand of a tap is fetched once and applied to every channel that has a nonzero there:
// one 16-byte LDS read feeds four multiply-adds per such channel instead of four in total.  Every
// channel still receives its products in ascending column order starting from the bias, so the
// results are bit-identical to the per-row kernels and to the reference's.
//
// The kernel is the LDS-windowed convolution (conv.hip) with another step loop: the same tiles,
// input-channel chunks, double-buffered windows and lane layout; a wave accumulates the block's
// channels in 32 registers (4 batch entries x 8 channels).  Which accumulator a product goes to
// depends on the data, and is wave-uniform: the multiply-adds run with the destination and the
// addend register-indexed (VGPR index mode: M0 holds the offset), M0 written from the stream
// before each group of four.  The stream is a sequence of records of fixed shape -- one tap and
// two (accumulator, weight) slots; a tap used by more channels takes several records, an unused
// slot multiplies -0 into a spare accumulator -- so the loop has no data-dependent branch.  Records
// arrive through scalar loads, four per load and one load ahead; the LDS reads of four records
// are issued while the previous four's multiply-adds run.
#include "conv_internal.h"

#include <algorithm>
#include <cstring>
#include <new>
#include <vector>

// ------------------------------------------------------------------ the format, as uploaded

extern "C" so_status so_rbm_upload(so_ctx *ctx, uint32_t M, uint32_t N, uint32_t Ct_max, uint32_t nblocks,
                                   const uint32_t *block_union, const uint32_t *krel, const uint32_t *colptr,
                                   const uint16_t *pair_row, const float *pair_w, so_rbm **out)
{
    SO_REQUIRE(ctx && out, "so_rbm_upload: null argument");
    *out = nullptr;
    SO_REQUIRE(Ct_max >= 1 && Ct_max <= 65535, "so_rbm_upload: Ct_max must be in 1..65535");
    SO_REQUIRE(nblocks == so_ceil_div(M, Ct_max), "so_rbm_upload: %u rows in blocks of %u are %u blocks, not %u", M, Ct_max,
               so_ceil_div(M, Ct_max), nblocks);
    SO_REQUIRE(block_union != nullptr && colptr != nullptr, "so_rbm_upload: block_union/colptr is null");
    SO_REQUIRE(block_union[0] == 0 && colptr[0] == 0, "so_rbm_upload: block_union and colptr must start at 0");
    const uint32_t U = block_union[nblocks];
    SO_REQUIRE(U == 0 || krel != nullptr, "so_rbm_upload: krel is null");
    // the pair arrays are read below: they must be there as soon as any union column claims a pair.  colptr has
    // U + 1 entries by contract; what it says is checked entry by entry before it is used as an index.
    bool any_pair = false;
    for (uint32_t u = 0; u < U && !any_pair; ++u) any_pair = colptr[u + 1] != colptr[u];
    SO_REQUIRE(!any_pair || (pair_row && pair_w), "so_rbm_upload: pair_row/pair_w is null");
    // every union column names a column of the matrix, columns ascend inside a block, every column
    // has at least one pair, the rows of a column ascend and lie inside the block
    for (uint32_t b = 0; b < nblocks; ++b) {
        if (block_union[b + 1] < block_union[b]) { so_set_error("so_rbm_upload: block_union decreases at block %u", b); return SO_ERR_BOUNDS; }
        const uint32_t rows = std::min(Ct_max, M - b * Ct_max);
        for (uint32_t u = block_union[b]; u < block_union[b + 1]; ++u) {
            if (krel[u] >= N) { so_set_error("so_rbm_upload: krel[%u] = %u is not below N = %u", u, krel[u], N); return SO_ERR_BOUNDS; }
            if (u > block_union[b] && krel[u] <= krel[u - 1]) { so_set_error("so_rbm_upload: union columns of block %u do not ascend at %u", b, u); return SO_ERR_BOUNDS; }
            if (colptr[u + 1] <= colptr[u]) { so_set_error("so_rbm_upload: union column %u has no pair", u); return SO_ERR_BOUNDS; }
            if (colptr[u + 1] - colptr[u] > rows) { so_set_error("so_rbm_upload: union column %u has more pairs than the block has rows", u); return SO_ERR_BOUNDS; }
            for (uint32_t p = colptr[u]; p < colptr[u + 1]; ++p) {
                if (pair_row[p] >= rows) { so_set_error("so_rbm_upload: pair %u names row %u of a block of %u", p, pair_row[p], rows); return SO_ERR_BOUNDS; }
                if (p > colptr[u] && pair_row[p] <= pair_row[p - 1]) { so_set_error("so_rbm_upload: rows of union column %u do not ascend", u); return SO_ERR_BOUNDS; }
            }
        }
    }
    const uint32_t P = colptr[U];
    SO_REQUIRE(P == 0 || (pair_row && pair_w), "so_rbm_upload: pair_row/pair_w is null");
    so_rbm *R = new (std::nothrow) so_rbm();
    if (!R) { so_set_error("so_rbm_upload: host allocation failed"); return SO_ERR_OOM; }
    R->M = M; R->N = N; R->Ct_max = Ct_max; R->nblocks = nblocks;
    R->block_union.assign(block_union, block_union + nblocks + 1);
    R->krel.assign(krel, krel + U);
    R->colptr.assign(colptr, colptr + U + 1);
    R->pair_row.assign(pair_row, pair_row + P);
    R->pair_w.assign(pair_w, pair_w + P);
    *out = R;
    return SO_OK;
}

extern "C" so_status so_rbm_free(so_ctx *ctx, so_rbm *R)
{
    if (!R) return SO_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    delete R;
    return SO_OK;
}

extern "C" so_status so_rbm_dims(const so_rbm *R, uint32_t *M, uint32_t *N, uint32_t *Ct_max, uint32_t *nblocks,
                                 uint64_t *total_union, uint64_t *total_pairs)
{
    SO_REQUIRE(R != nullptr, "so_rbm_dims: R is null");
    if (M) *M = R->M;
    if (N) *N = R->N;
    if (Ct_max) *Ct_max = R->Ct_max;
    if (nblocks) *nblocks = R->nblocks;
    if (total_union) *total_union = R->krel.size();
    if (total_pairs) *total_pairs = R->pair_w.size();
    return SO_OK;
}

// ------------------------------------------------------------------ the kernel

namespace {

constexpr uint32_t kRbmRows = 8;            // most rows of a block the kernel's accumulators hold
constexpr uint32_t kRbmSlots = 2;           // (accumulator, weight) slots of a record
constexpr uint32_t kRbmSetRecords = 4;      // records per scalar load
constexpr uint32_t kRbmTrash = 4 * kRbmRows;   // register offset of the spare accumulator
constexpr uint32_t kRbmIndexMode = 0xC000;  // M0[15:12]: index the destination (which a multiply-accumulate also reads)
constexpr uint32_t kRbmSetBytes = 64;       // four records of 4 dwords
constexpr int kRbmMaxPerThread = 5;         // float4 window elements a thread copies per chunk

typedef float f32x32 __attribute__((ext_vector_type(32)));

// One record: { pixel offset (inside the chunk's window) of the tap of the record one set further
// on, the two weights, the two M0 values (low and high half) }.
struct RbmRecord { uint32_t off_next, w0, w1, h01; };
static_assert(sizeof(RbmRecord) * kRbmSetRecords == kRbmSetBytes, "a set is 16 dwords");

// Registers of the step loop (fixed, because index mode offsets the register NUMBER of the
// accumulators): v[48:79] the 8 x 4 accumulators, v[80:83] the spare one, v[84:99] and v[100:115]
// the two sets of four operands, s[36:51] and s[52:67] the two sets of records, s[34:35] the stream.
//
// The multiply-adds of one record: M0 <- accumulator offset (and the index mode bits), then
// acc[M0 + j] += w * x[j] (fused) for the lane's four batch entries; twice.
#define RBM_RECORD(W0, W1, H, X0, X1, X2, X3)         \
    "s_mov_b32 m0, s" #H "\n\t"                       \
    "v_fmac_f32 v48, s" #W0 ", v" #X0 "\n\t"          \
    "v_fmac_f32 v49, s" #W0 ", v" #X1 "\n\t"          \
    "v_fmac_f32 v50, s" #W0 ", v" #X2 "\n\t"          \
    "v_fmac_f32 v51, s" #W0 ", v" #X3 "\n\t"          \
    "s_lshr_b32 m0, s" #H ", 16\n\t"                  \
    "v_fmac_f32 v48, s" #W1 ", v" #X0 "\n\t"          \
    "v_fmac_f32 v49, s" #W1 ", v" #X1 "\n\t"          \
    "v_fmac_f32 v50, s" #W1 ", v" #X2 "\n\t"          \
    "v_fmac_f32 v51, s" #W1 ", v" #X3 "\n\t"

// Half an iteration: the set in s[S0 .. S0+15] and the operands in v[XA .. XA+15] are consumed, the
// next set goes to s[TLO:THI] and the next operands to v[XB .. XB+15].
#define RBM_HALF(S0, S1, S2, S3, S4, S5, S6, S7, S8, S9, S10, S11, S12, S13, S14, S15, TLO, THI,                 \
                 XA0, XA1, XA2, XA3, XA4, XA5, XA6, XA7, XA8, XA9, XA10, XA11, XA12, XA13, XA14, XA15,           \
                 XB0, XB3, XB4, XB7, XB8, XB11, XB12, XB15)                                                      \
    "s_waitcnt lgkmcnt(0)\n\t"                                                      \
    "s_load_dwordx16 s[" #TLO ":" #THI "], s[34:35], 0x0\n\t"                       \
    "s_add_u32 s34, s34, 64\n\t"                                                    \
    "s_addc_u32 s35, s35, 0\n\t"                                                    \
    "s_mov_b32 m0, 0\n\t"                                                           \
    "v_lshl_add_u32 %[va0], s" #S0 ", %[shift], %[vbase]\n\t"                       \
    "v_lshl_add_u32 %[va1], s" #S4 ", %[shift], %[vbase]\n\t"                       \
    "v_lshl_add_u32 %[va2], s" #S8 ", %[shift], %[vbase]\n\t"                       \
    "v_lshl_add_u32 %[va3], s" #S12 ", %[shift], %[vbase]\n\t"                      \
    "ds_read_b128 v[" #XB0 ":" #XB3 "], %[va0]\n\t"                                 \
    "ds_read_b128 v[" #XB4 ":" #XB7 "], %[va1]\n\t"                                 \
    "ds_read_b128 v[" #XB8 ":" #XB11 "], %[va2]\n\t"                                \
    "ds_read_b128 v[" #XB12 ":" #XB15 "], %[va3]\n\t"                               \
    RBM_RECORD(S1, S2, S3, XA0, XA1, XA2, XA3)                                      \
    RBM_RECORD(S5, S6, S7, XA4, XA5, XA6, XA7)                                      \
    RBM_RECORD(S9, S10, S11, XA8, XA9, XA10, XA11)                                  \
    RBM_RECORD(S13, S14, S15, XA12, XA13, XA14, XA15)

// Runs `count` (>= 1) half-iterations over the sets at `sets`: acc[4*c + j] collects channel c,
// batch entry j.  vbase = this lane's byte address of the window's first pixel in LDS.
template <int SHIFT>
__device__ __forceinline__ void rbm_steps(f32x32 &acc, const int4 *sets, uint32_t count, uint32_t vbase)
{
    uint32_t va0, va1, va2, va3;
    asm volatile(
        "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
        "s_add_u32 s34, s34, 64\n\t"
        "s_addc_u32 s35, s35, 0\n\t"
        "s_set_gpr_idx_on 0, 0x0\n"
        "L_rbm_a_%=:\n\t"
        RBM_HALF(36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47, 48, 49, 50, 51, 52, 67,
                 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95, 96, 97, 98, 99,
                 100, 103, 104, 107, 108, 111, 112, 115)
        "s_sub_u32 %[cnt], %[cnt], 1\n\t"
        "s_cmp_eq_u32 %[cnt], 0\n\t"
        "s_cbranch_scc1 L_rbm_end_%=\n\t"
        RBM_HALF(52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63, 64, 65, 66, 67, 36, 51,
                 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111, 112, 113, 114, 115,
                 84, 87, 88, 91, 92, 95, 96, 99)
        "s_sub_u32 %[cnt], %[cnt], 1\n\t"
        "s_cmp_lg_u32 %[cnt], 0\n\t"
        "s_cbranch_scc1 L_rbm_a_%=\n"
        "L_rbm_end_%=:\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "s_mov_b32 m0, 0\n\t"
        "s_set_gpr_idx_off\n\t"
        : "+{v[48:79]}"(acc), [va0] "=&v"(va0), [va1] "=&v"(va1), [va2] "=&v"(va2), [va3] "=&v"(va3), [cnt] "+s"(count), "+{s[34:35]}"(sets)
        : [vbase] "v"(vbase), [shift] "n"(SHIFT)
        : "memory", "scc", "m0",
          "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95",
          "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107",
          "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115",
          "s36", "s37", "s38", "s39", "s40", "s41", "s42", "s43", "s44", "s45", "s46", "s47", "s48", "s49", "s50", "s51",
          "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67");
}

// Brings `lines` 64-byte lines from `p` on into the scalar cache: one scalar load per line, all in
// flight together, then one wait.  The step loop's own scalar loads then hit, which shortens the wait
// they share with the LDS reads (measured: 56x56x64 layer at batch 32 from 67 to 64 us, 7x7 stem from
// 98 to 89 us).
__device__ __forceinline__ void rbm_touch(const int4 *p, uint32_t lines, uint32_t part, uint32_t parts)
{
    // in groups of four lines (up to three past the range: the stream ends with padding sets); the
    // waves that walk the same stream -- the pixel groups of a block -- take every parts-th group each
    uint32_t groups = (lines + 3u) / 4u, sink;
    if (groups <= part) return;
    groups = (groups - part + parts - 1u) / parts;
    p += 16u * part;
    const uint32_t stride = 256u * parts;
    asm volatile(
        "L_rbm_touch_%=:\n\t"
        "s_load_dword %[d], s[34:35], 0x0\n\t"
        "s_load_dword %[d], s[34:35], 0x40\n\t"
        "s_load_dword %[d], s[34:35], 0x80\n\t"
        "s_load_dword %[d], s[34:35], 0xc0\n\t"
        "s_add_u32 s34, s34, %[st]\n\t"
        "s_addc_u32 s35, s35, 0\n\t"
        "s_sub_u32 %[n], %[n], 1\n\t"
        "s_cmp_lg_u32 %[n], 0\n\t"
        "s_cbranch_scc1 L_rbm_touch_%=\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        : [d] "=&s"(sink), "+{s[34:35]}"(p), [n] "+s"(groups)
        : [st] "s"(stride)
        : "scc");
}

template <int LPP, int ACT>
__global__ __launch_bounds__(kWinThreads)
void conv2d_rbm_kernel(const int4 *__restrict__ sets, const uint32_t *__restrict__ gbase,
                       const uint32_t *__restrict__ counts, WinArgs a, so_conv_geom g, uint32_t ct,
                       const float *__restrict__ X, uint32_t B, const float *__restrict__ bias,
                       const float *__restrict__ resid, float *__restrict__ Y)
{
    extern __shared__ float4 win_lds[];
    constexpr uint32_t BT = LPP * 4, PPW = 64 / LPP, SHIFT = (LPP == 4 ? 6 : LPP == 2 ? 5 : 4);
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t cgi = window_div(wave, a.pg, a.mPg), pgi = wave - cgi * a.pg;
    const uint32_t tile_y = window_div(blockIdx.x, a.tiles_x, a.mTilesX);
    const uint32_t th0 = tile_y * a.TH, tw0 = (blockIdx.x - tile_y * a.tiles_x) * a.TW;
    const uint32_t grp = blockIdx.y * a.cg + cgi;                    // block of output channels of this wave
    const uint32_t co0 = grp * ct;
    const uint32_t bz = blockIdx.z * BT;
    const bool computes = cgi < a.cg && grp < a.groups;              // the other waves only help copying
    const uint32_t gi = computes ? grp : 0u;

    // this lane's output pixel and its corner inside the window
    const uint32_t pl = pgi * PPW + lane / LPP, b4 = lane % LPP;
    const bool pvalid = pl < a.TH * a.TW;
    const uint32_t pc = window_slot_pixel(a, pl & 63u);          // slots beyond the tile repeat a pixel of their group
    const uint32_t ty = window_div(pc, a.TW, a.mTW), tx = pc - ty * a.TW;
    const bool live = computes && pvalid && th0 + ty < g.H_out && tw0 + tx < g.W_out;
    const uint32_t lanebase = ((ty * a.sth * a.IW + tx * a.stw) << SHIFT) + b4 * 16u;   // bytes
    const uint32_t buf_bytes = a.buf_f4 * 16u;

    // window elements this thread copies: element e = tid + k*1024 is float4 (cl, ih, iw, b4)
    int32_t goff[kRbmMaxPerThread];      // float offset from the chunk's first channel; -1: outside the image
    uint32_t gcl[kRbmMaxPerThread];      // channel inside the chunk; 0xffffffff: no such element
#pragma unroll
    for (int k = 0; k < kRbmMaxPerThread; ++k) {
        const uint32_t e = tid + (uint32_t)k * kWinThreads;
        goff[k] = -1;
        gcl[k] = 0xffffffffu;
        if (e < a.win_f4) {
            const uint32_t eb = e % LPP, px = e / LPP;
            const uint32_t rest = window_div(px, a.IW, a.mIW), iw = px - rest * a.IW;
            const uint32_t cl = window_div(rest, a.IH, a.mIH), ih = rest - cl * a.IH;
            const int32_t gh = (int32_t)(th0 * g.stride_h + ih * a.sbh) - (int32_t)g.pad_h;
            const int32_t gw = (int32_t)(tw0 * g.stride_w + iw * a.sbw) - (int32_t)g.pad_w;
            gcl[k] = cl;
            if ((uint32_t)gh < g.H_in && (uint32_t)gw < g.W_in)
                goff[k] = (int32_t)(((cl * g.H_in + (uint32_t)gh) * g.W_in + (uint32_t)gw) * B + bz + eb * 4u);
        }
    }
    const size_t chunk_floats = (size_t)a.cc * g.H_in * g.W_in * B;

    float4 xr[kRbmMaxPerThread];
    auto fetch_window = [&](uint32_t t) {
        const float *__restrict__ Xc = X + (size_t)t * chunk_floats;
        const uint32_t cleft = g.Cin - t * a.cc;                       // channels left from this chunk on
#pragma unroll
        for (int k = 0; k < kRbmMaxPerThread; ++k) {
            xr[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (goff[k] >= 0 && gcl[k] < cleft) xr[k] = *reinterpret_cast<const float4 *>(Xc + goff[k]);
        }
    };
    auto store_window = [&](uint32_t buf) {
#pragma unroll
        for (int k = 0; k < kRbmMaxPerThread; ++k)
            if (gcl[k] != 0xffffffffu) win_lds[buf * a.buf_f4 + tid + (uint32_t)k * kWinThreads] = xr[k];
    };

    f32x32 acc;
#pragma unroll
    for (int c = 0; c < (int)kRbmRows; ++c) {
        const float b0 = (bias && computes && (uint32_t)c < ct && co0 + c < g.Cout) ? bias[co0 + c] : 0.0f;
        acc[4 * c] = acc[4 * c + 1] = acc[4 * c + 2] = acc[4 * c + 3] = b0;
    }

    // the all-zero plane behind each window buffer (the taps of padding records point into it)
    for (uint32_t i = tid; i < a.buf_f4 - a.win_f4; i += kWinThreads) {
        win_lds[a.win_f4 + i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (a.nbuf == 2) win_lds[a.buf_f4 + a.win_f4 + i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    fetch_window(0);
    store_window(0);

    const int4 *__restrict__ sp = sets + (size_t)gbase[gi] * (kRbmSetBytes / 16);
    const uint32_t *__restrict__ cp = counts + (size_t)gi * a.nch;
    {
        const uint32_t n0 = computes ? __builtin_amdgcn_readfirstlane(cp[0]) : 0u;
        if (n0) rbm_touch(sp, n0 + 1u, pgi, a.pg);   // a set is one line; the loop requests one set past the last
    }
    __syncthreads();

    for (uint32_t t = 0; t < a.nch; ++t) {
        const bool more = t + 1 < a.nch;
        if (more) fetch_window(t + 1);
        const uint32_t cur_buf = a.nbuf == 2 ? (t & 1u) : 0u;
        const uint32_t n = computes ? __builtin_amdgcn_readfirstlane(cp[t]) : 0u;
        if (n != 0u) {
            rbm_steps<(int)SHIFT>(acc, sp, n, lanebase + cur_buf * buf_bytes);
            sp += (size_t)n * (kRbmSetBytes / 16);
        }
        if (more) {                                  // the next chunk's sets, while the slower waves finish this one
            const uint32_t nn = computes ? __builtin_amdgcn_readfirstlane(cp[t + 1]) : 0u;
            if (nn) rbm_touch(sp, nn + 1u, pgi, a.pg);
        }
        if (a.nbuf == 2) {
            if (more) store_window(cur_buf ^ 1u);
            __syncthreads();
        } else {
            __syncthreads();                       // every wave has finished reading the only buffer
            if (more) store_window(0);
            __syncthreads();
        }
    }

    if (live) {
        const uint32_t ho = th0 + ty, wo = tw0 + tx;
#pragma unroll
        for (int c = 0; c < (int)kRbmRows; ++c) {
            const uint32_t co = co0 + c;
            if ((uint32_t)c < ct && co < g.Cout) {
                const size_t at = (((size_t)co * g.H_out + ho) * g.W_out + wo) * B + bz + b4 * 4u;
                float v0 = acc[4 * c], v1 = acc[4 * c + 1], v2 = acc[4 * c + 2], v3 = acc[4 * c + 3];
                if (resid) {             // conv + skip, then the activation
                    const float4 rv = *reinterpret_cast<const float4 *>(resid + at);
                    v0 += rv.x; v1 += rv.y; v2 += rv.z; v3 += rv.w;
                }
                float4 out;
                out.x = so_epilogue<ACT>(v0); out.y = so_epilogue<ACT>(v1);
                out.z = so_epilogue<ACT>(v2); out.w = so_epilogue<ACT>(v3);
                *reinterpret_cast<float4 *>(Y + at) = out;
            }
        }
    }
}

template <int LPP>
hipError_t rbm_allow_lds(so_ctx *ctx)
{
    hipError_t e = hipSuccess;
    const void *k[4] = {(const void *)conv2d_rbm_kernel<LPP, SO_ACT_NONE>, (const void *)conv2d_rbm_kernel<LPP, SO_ACT_RELU>,
                        (const void *)conv2d_rbm_kernel<LPP, SO_ACT_SIGMOID>, (const void *)conv2d_rbm_kernel<LPP, SO_ACT_TANH>};
    for (const void *f : k)
        if (e == hipSuccess) e = so_allow_big_lds(ctx, f);
    return e;
}

template <int LPP>
void rbm_launch_act(so_ctx *ctx, const so_conv_plan *plan, const WinArgs &a, dim3 grid, size_t lds,
                    const float *dX, uint32_t B, const float *dBias, const float *dResid, float *dY, int act)
{
    const so_conv_rbm &r = plan->rbm;
#define SO_RBM_LAUNCH(A)                                                                              \
    conv2d_rbm_kernel<LPP, A><<<grid, kWinThreads, lds, ctx->stream>>>(                               \
        reinterpret_cast<const int4 *>(r.d_sets), r.d_gbase, r.d_counts, a, plan->g, r.src->Ct_max,   \
        dX, B, dBias, dResid, dY)
    switch (act) {
    case SO_ACT_RELU:    SO_RBM_LAUNCH(SO_ACT_RELU); break;
    case SO_ACT_SIGMOID: SO_RBM_LAUNCH(SO_ACT_SIGMOID); break;
    case SO_ACT_TANH:    SO_RBM_LAUNCH(SO_ACT_TANH); break;
    default:             SO_RBM_LAUNCH(SO_ACT_NONE); break;
    }
#undef SO_RBM_LAUNCH
}

// A wave of this kernel owns a whole block of channels, so a launch has an eighth of the waves the
// per-row kernel can spread over the chip: it needs a grid that covers about three quarters of the
// compute units (28x28x128 at batch 32, 112 workgroups: 113 against 66 us).  With such a grid it is
// level with the per-row kernel on stride-1 layers (ResNet-18 shapes, 3x3: 56x56x64 at batch 32 64.4
// against 62.9 us, at batch 128 256 against 258; 28x28x128 at batch 128 224 against 219) and ahead
// on strided ones (7x7 stride-2 stem 87 against 99 us at batch 32, 299 against 339 at batch 128;
// 3x3 stride-2 56->28 at batch 64 71 against 80; 1x1 stride-2 18 against 19): it runs there.
bool rbm_pays(const so_ctx *ctx, const so_conv_geom &g, uint64_t workgroups)
{
    return 4ull * workgroups >= 3ull * (uint64_t)ctx->compute_units && (g.stride_h > 1 || g.stride_w > 1);
}

} // namespace

// ------------------------------------------------------------------ streams of a plan

void so_conv_rbm_release(so_conv_plan *plan)
{
    so_conv_rbm &r = plan->rbm;
    if (r.d_sets) (void)hipFree(r.d_sets);
    if (r.d_gbase) (void)hipFree(r.d_gbase);
    if (r.d_counts) (void)hipFree(r.d_counts);
    const so_rbm *src = r.src;
    r = so_conv_rbm();
    r.src = src;
}

// (Re)builds the record streams for the plan's current window (tile, channel chunks); leaves the
// plan without streams when it has no window layout or no attached format.
so_status so_conv_rbm_rebuild(so_ctx *ctx, so_conv_plan *plan)
{
    so_conv_rbm_release(plan);
    const so_rbm *R = plan->rbm.src;
    const so_conv_window &w = plan->win;
    if (!R || w.cc == 0) return SO_OK;
    const so_conv_geom &g = plan->g;
    const uint32_t kHW = g.kH * g.kW, zero_plane = w.cc * w.IH * w.IW;
    const uint32_t pad_h = kRbmIndexMode | kRbmTrash, pad_w = 0x80000000u;      // -0.0 into the spare accumulator
    const RbmRecord padrec{zero_plane, pad_w, pad_w, pad_h | (pad_h << 16)};

    std::vector<RbmRecord> stream;                 // all blocks, chunk after chunk
    std::vector<uint32_t> gbase(R->nblocks), counts((size_t)R->nblocks * w.nch, 0);
    std::vector<RbmRecord> recs;                   // records of one (block, chunk); off_next holds the record's own tap here
    uint64_t real_pairs = 0, slots = 0;
    for (uint32_t b = 0; b < R->nblocks; ++b) {
        gbase[b] = (uint32_t)(stream.size() / kRbmSetRecords);
        uint32_t u = R->block_union[b];
        const uint32_t u_end = R->block_union[b + 1];
        for (uint32_t t = 0; t < w.nch; ++t) {
            recs.clear();
            for (; u < u_end && R->krel[u] / kHW / w.cc == t; ++u) {
                const uint32_t k = R->krel[u];
                const uint32_t cin = k / kHW, kh = (k / g.kW) % g.kH, kw = k % g.kW;
                const uint32_t off = ((cin - t * w.cc) * w.IH + kh * g.dil_h) * w.IW + kw * g.dil_w;
                for (uint32_t p = R->colptr[u]; p < R->colptr[u + 1]; p += kRbmSlots) {
                    RbmRecord rec = padrec;
                    rec.off_next = off;
                    std::memcpy(&rec.w0, &R->pair_w[p], 4);
                    rec.h01 = (rec.h01 & 0xffff0000u) | kRbmIndexMode | (4u * R->pair_row[p]);
                    ++real_pairs;
                    if (p + 1 < R->colptr[u + 1]) {
                        std::memcpy(&rec.w1, &R->pair_w[p + 1], 4);
                        rec.h01 = (rec.h01 & 0xffffu) | ((kRbmIndexMode | (4u * R->pair_row[p + 1])) << 16);
                        ++real_pairs;
                    }
                    recs.push_back(rec);
                }
            }
            if (recs.empty()) continue;
            while (recs.size() % kRbmSetRecords) recs.push_back(padrec);
            slots += recs.size() * kRbmSlots;
            // set j carries the taps of records 4j .. 4j+3 (fetched during half-iteration j) and the
            // weights of records 4j-4 .. 4j-1 (whose operands half-iteration j-1 fetched)
            const size_t nsets = recs.size() / kRbmSetRecords + 1;
            for (size_t j = 0; j < nsets; ++j)
                for (size_t k = 0; k < kRbmSetRecords; ++k) {
                    RbmRecord out = padrec;
                    if (kRbmSetRecords * j + k < recs.size()) out.off_next = recs[kRbmSetRecords * j + k].off_next;
                    if (j >= 1) {
                        const RbmRecord &from = recs[kRbmSetRecords * (j - 1) + k];
                        out.w0 = from.w0; out.w1 = from.w1; out.h01 = from.h01;
                    }
                    stream.push_back(out);
                }
            counts[(size_t)b * w.nch + t] = (uint32_t)nsets;
        }
        if (stream.size() / kRbmSetRecords > 0x7ffffff0ull) { so_set_error("so_conv_plan_set_rbm: stream too large"); return SO_ERR_INVALID; }
    }
    // the loop requests one set past the last one it uses, the touches reach up to three lines further
    for (uint32_t k = 0; k < 4 * kRbmSetRecords; ++k) stream.push_back(padrec);

    hipError_t e = rbm_allow_lds<4>(ctx);
    if (e == hipSuccess) e = rbm_allow_lds<2>(ctx);
    if (e == hipSuccess) e = rbm_allow_lds<1>(ctx);
    if (e != hipSuccess) { so_set_error("so_conv_plan_set_rbm: hipFuncSetAttribute failed: %s", hipGetErrorString(e)); return SO_ERR_HIP; }
    void *d1 = nullptr, *d2 = nullptr, *d3 = nullptr;
    so_status s = so_malloc(ctx, stream.size() * sizeof(RbmRecord), &d1);
    if (s == SO_OK) s = so_h2d(ctx, d1, stream.data(), stream.size() * sizeof(RbmRecord));
    if (s == SO_OK) s = so_malloc(ctx, std::max<size_t>(1, gbase.size()) * sizeof(uint32_t), &d2);
    if (s == SO_OK && !gbase.empty()) s = so_h2d(ctx, d2, gbase.data(), gbase.size() * sizeof(uint32_t));
    if (s == SO_OK) s = so_malloc(ctx, std::max<size_t>(1, counts.size()) * sizeof(uint32_t), &d3);
    if (s == SO_OK && !counts.empty()) s = so_h2d(ctx, d3, counts.data(), counts.size() * sizeof(uint32_t));
    if (s != SO_OK) {
        if (d1) (void)hipFree(d1);
        if (d2) (void)hipFree(d2);
        if (d3) (void)hipFree(d3);
        return s;
    }
    so_conv_rbm &r = plan->rbm;
    r.d_sets = d1;
    r.d_gbase = (uint32_t *)d2;
    r.d_counts = (uint32_t *)d3;
    r.total_sets = stream.size() / kRbmSetRecords;
    r.real_pairs = real_pairs;
    r.slots = slots;
    return SO_OK;
}

extern "C" so_status so_conv_plan_set_rbm(so_ctx *ctx, so_conv_plan *plan, const so_rbm *R)
{
    SO_REQUIRE(ctx && plan, "so_conv_plan_set_rbm: null argument");
    SO_REQUIRE(!ctx->capturing, "so_conv_plan_set_rbm: not allowed while a graph is being recorded");
    SO_HIP(hipStreamSynchronize(ctx->stream));      // no launch may still be reading the old streams
    if (R) {
        SO_REQUIRE(R->M == plan->g.Cout && (uint64_t)R->N == (uint64_t)plan->g.Cin * plan->g.kH * plan->g.kW,
                   "so_conv_plan_set_rbm: the format is %u x %u, the plan's weights are %u x %llu", R->M, R->N, plan->g.Cout,
                   (unsigned long long)plan->g.Cin * plan->g.kH * plan->g.kW);
        SO_REQUIRE(R->Ct_max <= kRbmRows, "so_conv_plan_set_rbm: blocks of %u rows; the kernel holds at most %u", R->Ct_max, kRbmRows);
    }
    so_conv_rbm_release(plan);
    plan->rbm.src = R;
    return so_conv_rbm_rebuild(ctx, plan);
}

extern "C" so_status so_conv_plan_rbm_info(const so_conv_plan *plan, uint64_t out[4])
{
    SO_REQUIRE(plan && out, "so_conv_plan_rbm_info: null argument");
    const so_conv_rbm &r = plan->rbm;
    out[0] = r.d_sets ? r.total_sets : 0;
    out[1] = r.d_sets ? r.real_pairs : 0;
    out[2] = r.d_sets ? r.slots : 0;
    out[3] = r.d_sets ? kRbmSlots : 0;
    return SO_OK;
}

// Launches the RBM kernel if the plan carries its streams, the batch suits the windowed layout and
// (unless `forced`) the launch is one on which it beats the per-row windowed kernel; *done says
// whether it did.
so_status so_conv_rbm_launch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B, const float *dBias,
                             const float *dResid, float *dY, int act, bool forced, bool *done)
{
    *done = false;
    const so_conv_window &w = plan->win;
    const so_conv_rbm &r = plan->rbm;
    const uint32_t LPP = window_lpp(B);
    if (!r.d_sets || w.cc == 0 || LPP == 0) return SO_OK;
    const uint32_t PPW = 64 / LPP;
    WinArgs a;
    a.TH = w.TH; a.TW = w.TW; a.IH = w.IH; a.IW = w.IW; a.cc = w.cc; a.nch = w.nch; a.tiles_x = w.tiles_x;
    a.groups = r.src->nblocks;
    a.pg = so_ceil_div(w.TH * w.TW, PPW);
    a.cg = 16 / a.pg;
    a.win_f4 = w.cc * w.IH * w.IW * LPP;
    a.buf_f4 = (w.cc + 1) * w.IH * w.IW * LPP;
    a.nbuf = w.nch > 1 ? 2u : 1u;
    a.sth = window_step(plan->g.kH, plan->g.stride_h); a.stw = window_step(plan->g.kW, plan->g.stride_w);
    a.sbh = window_subsample(plan->g.kH, plan->g.stride_h); a.sbw = window_subsample(plan->g.kW, plan->g.stride_w);
    window_pixel_order(a, LPP);
    a.mIW = window_magic(a.IW); a.mIH = window_magic(a.IH); a.mTW = window_magic(a.TW);
    a.mTilesX = window_magic(a.tiles_x); a.mPg = window_magic(a.pg);
    a.ws = so_lds::wait_status{0, nullptr};      // this kernel synchronises with barriers
    const size_t lds = (size_t)a.nbuf * a.buf_f4 * 16;
    // a layout whose chunks were sized for a smaller batch tile than this batch's does not fit
    if (LPP > w.lpp && (lds > (size_t)ctx->max_lds_bytes || a.win_f4 > (uint32_t)kRbmMaxPerThread * kWinThreads)) return SO_OK;
    if (a.win_f4 > (uint32_t)kRbmMaxPerThread * kWinThreads) return SO_OK;      // this kernel copies at most that many elements per thread
    const dim3 grid(w.tiles_x * w.tiles_y, so_ceil_div(a.groups, a.cg), B / (4 * LPP));
    if (grid.y > 65535u || grid.z > 65535u) return SO_OK;
    if (!forced && !rbm_pays(ctx, plan->g, (uint64_t)grid.x * grid.y * grid.z)) return SO_OK;
    switch (LPP) {
    case 4:  rbm_launch_act<4>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    case 2:  rbm_launch_act<2>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    default: rbm_launch_act<1>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    }
    *done = true;
    return SO_OK;
}
