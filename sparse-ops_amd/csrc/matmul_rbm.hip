// Row-block-merged (RBM) matmul: layout SO_LAYOUT_RBM, its builder and its kernel.
//
// The reference's blocked-CSC idea (include/rbm_conv.hpp:8-27, src/layers/rbm_conv.cpp:7-73;
// kernel loop src/layers/conv_kernels.cpp:96-123) applied to Y = E * X: rows are taken in blocks,
// a block's used columns are walked once, and the X row segment of a column is loaded once --
// one coalesced 256-byte load, a dword per lane -- and multiplied into every row of the block
// that has a nonzero there.  Nothing is staged in LDS, no operand is re-read per row, and the
// multiply-adds are plain fp32 FMAs whose accumulator is picked by VGPR index mode.
//
// Decomposition.  A workgroup of 12 waves owns a tile of 128 rows x 64 dense columns (lane =
// column) and 1/ksplit of the block's columns; every wave holds the tile's 128 accumulators
// and works through its own share of the columns ("stream"), so a tile is the sum of 12 x ksplit
// partial tiles: the 12 of a workgroup are added through LDS, the ksplit workgroups of a tile
// meet in memory -- each stores its partial tile, the last one to arrive (a counter per tile) adds
// them in a fixed order, applies bias and activation and writes Y.  No workgroup ever waits for
// another.
//
// Streams.  The step loop is straight-line code (matmul_rbm_steps.inc, written by
// gen_matmul_rbm_steps.py): an iteration handles four columns that all have the same number s of
// (row, weight) pairs, one code body per s ("class", 6 .. 16).  The builder therefore cuts a
// column with more than 16 pairs into equal parts, pads every part to its class with (spare
// accumulator, -0) pairs, hands the parts of a class out to the block's streams four at a time so
// that every stream gets the same number of iterations of every class, and moves what is left
// over to the next class (one padding pair each).  The order of a stream's columns is free --
// sums are taken in that order, which is why this kernel is accurate to fp32 round-off
// (|y - ref| <= 1e-5 * max|ref|) instead of bit-identical to the reference's row order.  Streams
// start at different classes so that the waves of a SIMD do not all switch code at once.
//
// Results are deterministic: the same handle, X and C give the same bits on every launch.
#include "so_internal.h"

#include "matmul_rbm_steps.inc"

#include <algorithm>
#include <cstring>
#include <new>
#include <utility>
#include <vector>

namespace {

constexpr uint32_t RB = so_rbmm::kBlockRows, NW = so_rbmm::kWaves, SLOTS = 4, MAXP = 16, CMIN = 6, NCLASS = 11;
constexpr uint32_t RECDW = 64, RECBYTES = RECDW * 4, TRASH = RB, IDXMODE = 0xC000, TAILRECS = 5;
constexpr uint32_t GROUPS = RB / 4;                       // groups of 4 rows in a tile
constexpr uint32_t PASS_GROUPS = NW;                      // groups reduced per pass: one per wave
constexpr uint32_t LDS_BYTES = NW * PASS_GROUPS * 64 * 16 + 16;

struct Part {
    uint32_t j;                                           // column of E = row of X
    std::vector<std::pair<uint32_t, float>> pr;           // (row inside the block, weight)
};

typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define SO_RBMM_VCLOB "v132", "v133", "v134", "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", \
                      "v147", "v148", "v149", "v150", "v151", "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", \
                      "v162", "v163", "v164", "v165"
#define SO_RBMM_SCLOB "s24", "s25", "s26", "s27", "s28", "s29", "s30", "s31", \
                      "s32", "s33", "s34", "s35", "s36", "s37", "s38", "s39", "s40", "s41", "s42", "s43", "s44", "s45", "s46", "s47", \
                      "s48", "s49", "s50", "s51", "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", \
                      "s64", "s65", "s66", "s67", "s68", "s69", "s70", "s71", "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", \
                      "s80", "s81", "s82", "s83", "s84", "s85", "s86", "s87", "s88", "s89", "s90", "s91", "s92", "s93", "s94", "s95"

template <int ACT>
__global__ __launch_bounds__(NW * 64)
void ellpack_matmul_rbm_kernel(const uint32_t *__restrict__ hdr, const uint32_t *__restrict__ rec, const float *__restrict__ wts,
                               uint64_t nrec, uint32_t m, uint32_t n, uint32_t nb, uint32_t ksplit,
                               const float *__restrict__ X, uint32_t C, const float *__restrict__ bias, float *__restrict__ Y,
                               uint32_t nslabs, float *__restrict__ part, uint32_t *__restrict__ counters)
{
    extern __shared__ __attribute__((aligned(16))) float red[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup ids go round the 8 XCDs.  An XCD works on one part of K only (part kh of every
    // stream set covers a contiguous range of columns, so its L2 holds 1/ksplit of X), and the
    // nslabs workgroups that walk the same records take consecutive ids on it, so the records and
    // weights reach that L2 once.
    const uint32_t xcd = blockIdx.x & 7u, q = blockIdx.x >> 3, groups = 8u / ksplit;
    const uint32_t slab = q % nslabs, kh = xcd % ksplit, b = (q / nslabs) * groups + xcd / ksplit;
    if (b >= nb) return;
    const uint32_t hdr_dw = 8u + NW * ksplit * 2u;
    const uint32_t *h = hdr + (size_t)b * hdr_dw;
    const uint32_t q0 = __builtin_amdgcn_readfirstlane(h[0]), q1 = __builtin_amdgcn_readfirstlane(h[1]), q2 = __builtin_amdgcn_readfirstlane(h[2]);
    const uint32_t q3 = __builtin_amdgcn_readfirstlane(h[3]), q4 = __builtin_amdgcn_readfirstlane(h[4]), q5 = __builtin_amdgcn_readfirstlane(h[5]);
    const uint32_t stream = kh * NW + wave;
    const uint32_t rec0 = __builtin_amdgcn_readfirstlane(h[8 + stream * 2]);
    uint32_t entry = __builtin_amdgcn_readfirstlane(h[8 + stream * 2 + 1]);
    const uint32_t *recp = rec + (size_t)rec0 * RECDW;
    // Buffer resources: loads beyond the range return zero, so the loads the loop requests past a
    // stream's end (it runs three iterations ahead) and a lane past the last column are harmless.
    u32x4 xr, wr;
    {
        const uint64_t xb = (uint64_t)X + (uint64_t)slab * 256u;
        const uint64_t xbytes = (uint64_t)n * C * 4u - (uint64_t)slab * 256u;
        xr[0] = (uint32_t)xb; xr[1] = (uint32_t)(xb >> 32) & 0xffffu; xr[2] = (uint32_t)std::min<uint64_t>(xbytes, 0xffffffffu); xr[3] = 0x00020000u;
        const uint64_t wb = (uint64_t)wts + (uint64_t)rec0 * RECBYTES;
        const uint64_t wbytes = (nrec - rec0) * RECBYTES;
        wr[0] = (uint32_t)wb; wr[1] = (uint32_t)(wb >> 32) & 0xffffu; wr[2] = (uint32_t)std::min<uint64_t>(wbytes, 0xffffffffu); wr[3] = 0x00020000u;
#pragma unroll
        for (int i = 0; i < 4; ++i) { xr[i] = __builtin_amdgcn_readfirstlane(xr[i]); wr[i] = __builtin_amdgcn_readfirstlane(wr[i]); }
    }
    f32x32 a0, a1, a2, a3;
#pragma unroll
    for (int i = 0; i < 32; ++i) { a0[i] = 0.f; a1[i] = 0.f; a2[i] = 0.f; a3[i] = 0.f; }
    uint32_t off = 0, cnt = 0, left = NCLASS;
    const uint32_t lane4 = lane * 4u, wlane = (lane & 15u) * 16u;
    asm volatile(SO_RBMM_STEPS_ASM
                 : "+{v[4:35]}"(a0), "+{v[36:67]}"(a1), "+{v[68:99]}"(a2), "+{v[100:131]}"(a3), "+{s18}"(off), "+{s20}"(cnt), "+{s21}"(left), "+{s22}"(entry)
                 : "{s2}"(q0), "{s3}"(q1), "{s4}"(q2), "{s5}"(q3), "{s6}"(q4), "{s7}"(q5), "{s[8:11]}"(xr), "{s[12:15]}"(wr), "{s[16:17]}"(recp),
                   "{v166}"(lane4), "{v167}"(wlane)
                 : "memory", "scc", "m0", SO_RBMM_VCLOB, SO_RBMM_SCLOB);

    // The 12 partial tiles of the workgroup, added through LDS: groups of 4 rows (one 16-byte
    // element per lane), 12 groups per pass, wave w adds group w of the pass over the 12 waves in
    // wave order.  The workgroup's partial tile, [group][lane][4 rows], goes to `part` (or, with
    // ksplit == 1, straight on to the epilogue).
    f32x4 *red4 = reinterpret_cast<f32x4 *>(red);
    const uint32_t col = slab * 64u + lane;
    const uint32_t tile = b * nslabs + slab;
    f32x4 *mine = reinterpret_cast<f32x4 *>(part) + ((size_t)tile * ksplit + kh) * GROUPS * 64;
    auto rows4 = [&](int g) -> f32x4 {
        const f32x32 &a = g < 8 ? a0 : g < 16 ? a1 : g < 24 ? a2 : a3;
        const int o = 4 * (g & 7);
        f32x4 v; v[0] = a[o]; v[1] = a[o + 1]; v[2] = a[o + 2]; v[3] = a[o + 3];
        return v;
    };
    auto finish = [&](uint32_t g, const f32x4 &s) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t row = b * RB + g * 4u + e;
            if (row < m && col < C) Y[(size_t)row * C + col] = so_epilogue<ACT>(s[e] + (bias ? bias[row] : 0.0f));
        }
    };
#pragma unroll
    for (int pass = 0; pass < 3; ++pass) {
        const int g0 = pass * (int)PASS_GROUPS, G = pass < 2 ? (int)PASS_GROUPS : (int)(GROUPS - 2 * PASS_GROUPS);
        if (pass) __syncthreads();
#pragma unroll
        for (int k = 0; k < (int)PASS_GROUPS; ++k) if (k < G) red4[(wave * PASS_GROUPS + k) * 64 + lane] = rows4(g0 + k);
        __syncthreads();
        if ((int)wave < G) {
            f32x4 s = red4[wave * 64 + lane];
#pragma unroll
            for (int w = 1; w < (int)NW; ++w) { const f32x4 v = red4[(w * PASS_GROUPS + wave) * 64 + lane]; s[0] += v[0]; s[1] += v[1]; s[2] += v[2]; s[3] += v[3]; }
            if (ksplit == 1) finish((uint32_t)g0 + wave, s);
            // sc1: written through to memory, whichever XCD the tile's other workgroups run on
            else asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(mine + (g0 + wave) * 64 + lane), "v"(s) : "memory");
        }
    }
    if (ksplit == 1) return;
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");       // this wave's part of the partial tile has been written
    __syncthreads();
    uint32_t *arrived = reinterpret_cast<uint32_t *>(red + NW * PASS_GROUPS * 64 * 4);
    if (tid == 0) *arrived = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*arrived != ksplit - 1) return;                      // the last workgroup of the tile to arrive finishes it
    if (tid == 0) __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
    // this wave's groups (w, w + 12, w + 24) of all partial tiles: every load is requested before the first is waited for
    const f32x4 *p = reinterpret_cast<const f32x4 *>(part) + (size_t)tile * ksplit * GROUPS * 64;
    constexpr int kMine = (GROUPS + NW - 1) / NW;
    f32x4 v[kMine][so_rbmm::kMaxSplit];
#pragma unroll
    for (int i = 0; i < kMine; ++i) {
        const uint32_t g = wave + (uint32_t)i * NW;
#pragma unroll
        for (int k = 0; k < (int)so_rbmm::kMaxSplit; ++k)
            if (g < GROUPS && (uint32_t)k < ksplit)
                asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[i][k]) : "v"(p + ((size_t)k * GROUPS + g) * 64 + lane) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
#pragma unroll
    for (int i = 0; i < kMine; ++i) {
        const uint32_t g = wave + (uint32_t)i * NW;
        if (g >= GROUPS) break;
        f32x4 s = v[i][0];
#pragma unroll
        for (int k = 1; k < (int)so_rbmm::kMaxSplit; ++k)
            if ((uint32_t)k < ksplit) { s[0] += v[i][k][0]; s[1] += v[i][k][1]; s[2] += v[i][k][2]; s[3] += v[i][k][3]; }
        finish(g, s);
    }
}

// The records address X rows by byte offset (row * pitch): written here for the pitch of the launch at hand,
// once per handle and pitch.
__global__ void rbmm_offsets_kernel(uint32_t *__restrict__ rec, const uint32_t *__restrict__ xrows, uint64_t nrec, uint32_t pitch)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nrec * 4) rec[(i >> 2) * RECDW + 32 + (i & 3)] = xrows[i] * pitch;
}

template <int ACT>
so_status launch_rbm(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C, const float *dBias, float *dY)
{
    const so_rbmm &R = E->rbmm;
    SO_HIP(so_allow_big_lds(ctx, (const void *)ellpack_matmul_rbm_kernel<ACT>));
    const uint32_t nslabs = so_ceil_div(C, 64);
    const uint32_t blocks = so_ceil_div(R.nb, 8 / R.ksplit) * 8 * nslabs;      // ksplit is 1, 2 or 4
    ellpack_matmul_rbm_kernel<ACT><<<blocks, NW * 64, LDS_BYTES, ctx->stream>>>(
        R.d_hdr, R.d_rec, R.d_w, R.nrec, E->m, E->n, R.nb, R.ksplit, dX, C, dBias, dY, nslabs, ctx->mm_part, ctx->mm_counters);
    return SO_OK;
}

} // namespace

// ------------------------------------------------------------------ the builder

so_status so_rbmm_build(so_ctx *ctx, so_ellpack *E, const float *Wd, const uint32_t *idx, const uint32_t *nnz)
{
    const uint32_t m = E->m, n = E->n, r = E->r;
    so_rbmm &R = E->rbmm;
    R.nb = so_ceil_div(m, RB);
    // Workgroups per tile: enough that a 256-column launch covers the chip, as long as every
    // stream still gets a few columns.
    uint32_t ks = 1;
    while (ks < so_rbmm::kMaxSplit && (uint64_t)R.nb * 4 * ks < (uint64_t)ctx->compute_units && (uint64_t)n >= 64ull * NW * ks) ks *= 2;
    if (ctx->tune.matmul_rbm_split == 1 || ctx->tune.matmul_rbm_split == 2 || ctx->tune.matmul_rbm_split == 4) ks = (uint32_t)ctx->tune.matmul_rbm_split;
    R.ksplit = ks;
    const uint32_t NS = NW * ks, per = NS * SLOTS, hdr_dw = 8 + NS * 2;
    std::vector<uint32_t> hdr((size_t)R.nb * hdr_dw, 0), rec, xrows;
    std::vector<float> w;
    rec.reserve((size_t)(E->total_nnz / 40 + (size_t)R.nb * NS * (TAILRECS + 8)) * RECDW);
    w.reserve(rec.capacity());
    std::vector<std::vector<std::pair<uint32_t, float>>> cols(n);
    std::vector<uint32_t> used;
    uint64_t slots_total = 0, parts_total = 0;
    const auto pad_pair = std::make_pair(TRASH, -0.0f);
    for (uint32_t b = 0; b < R.nb; ++b) {
        for (uint32_t j : used) cols[j].clear();
        used.clear();
        for (uint32_t i = b * RB; i < std::min(m, (b + 1) * RB); ++i)
            for (uint32_t k = 0; k < nnz[i]; ++k) {
                const uint32_t j = idx[(size_t)i * r + k];
                if (cols[j].empty()) used.push_back(j);
                cols[j].push_back({i - b * RB, Wd[(size_t)i * r + k]});
            }
        std::sort(used.begin(), used.end());
        // parts by class; the parts of one column stay next to each other (the second load of its X row hits L1)
        std::vector<std::vector<Part>> multi(MAXP + 1), single(MAXP + 1);
        for (uint32_t j : used) {
            const uint32_t c = (uint32_t)cols[j].size();
            const uint32_t np = so_ceil_div(c, MAXP), s = std::max(CMIN, so_ceil_div(c, np));
            for (uint32_t qn = 0; qn < np; ++qn) {
                Part pt; pt.j = j;
                for (uint32_t e = qn * s; e < std::min(c, (qn + 1) * s); ++e) pt.pr.push_back(cols[j][e]);
                pt.pr.resize(s, pad_pair);
                (np > 1 ? multi : single)[s].push_back(std::move(pt));
            }
        }
        std::vector<std::vector<Part>> cls(MAXP + 1);
        uint32_t q[MAXP + 1] = {0};
        std::vector<Part> carry;
        for (uint32_t s = CMIN; s <= MAXP; ++s) {
            std::vector<Part> L = std::move(multi[s]);
            for (auto &p : single[s]) L.push_back(std::move(p));
            for (auto &p : carry) { p.pr.push_back(pad_pair); L.push_back(std::move(p)); }
            carry.clear();
            std::stable_sort(L.begin(), L.end(), [](const Part &a, const Part &c) { return a.j < c.j; });
            if (s < MAXP) {                                       // what does not fill a round of all streams moves up a class
                const size_t keep = L.size() / per * per;
                for (size_t e = keep; e < L.size(); ++e) carry.push_back(std::move(L[e]));
                L.resize(keep);
            } else {
                while (L.size() % per) { Part d; d.j = 0; d.pr.assign(s, pad_pair); L.push_back(std::move(d)); }
            }
            if (L.size() / per > 0xffffu) { so_set_error("so_ellpack_upload: too many columns for the RBM layout"); return SO_ERR_INVALID; }
            q[s] = (uint32_t)(L.size() / per);
            cls[s] = std::move(L);
        }
        uint32_t *h = &hdr[(size_t)b * hdr_dw];
        for (uint32_t s = CMIN; s <= MAXP; ++s) h[(s - CMIN) / 2] |= q[s] << (16 * ((s - CMIN) % 2));
        for (uint32_t st = 0; st < NS; ++st) {
            const uint32_t entry = CMIN + st % NCLASS;
            if (rec.size() / RECDW > 0xfffffff0ull) { so_set_error("so_ellpack_upload: matrix too large for the RBM layout"); return SO_ERR_INVALID; }
            h[8 + st * 2] = (uint32_t)(rec.size() / RECDW);
            h[8 + st * 2 + 1] = entry;
            for (uint32_t v = 0; v < NCLASS; ++v) {
                const uint32_t s = CMIN + (entry - CMIN + v) % NCLASS;
                for (uint32_t it = 0; it < q[s]; ++it) {
                    // the class's parts are in column order: the kh-th of ksplit equal ranges belongs to the
                    // streams of part kh, dealt four per iteration over its NW streams
                    const size_t g = (size_t)(st / NW) * (cls[s].size() / ks) + ((size_t)it * NW + st % NW) * SLOTS;
                    uint32_t rd[RECDW] = {0};
                    const size_t wb = w.size();
                    for (uint32_t k = 0; k < SLOTS; ++k) {
                        const Part &pt = cls[s][g + k];
                        xrows.push_back(pt.j);
                        for (uint32_t p = 0; p < MAXP; ++p)
                            rd[8 * k + p / 2] |= (IDXMODE | (p < s ? pt.pr[p].first : TRASH)) << (16 * (p % 2));
                        for (uint32_t p = 0; p < s; ++p) w.push_back(pt.pr[p].second);
                    }
                    w.resize(wb + RECDW, -0.0f);
                    rec.insert(rec.end(), rd, rd + RECDW);
                    slots_total += SLOTS * s;
                    parts_total += SLOTS;
                }
            }
            for (uint32_t e = 0; e < TAILRECS; ++e) {             // what the loop requests past the stream's end
                uint32_t rd[RECDW] = {0};
                for (int k = 0; k < 32; ++k) rd[k] = (IDXMODE | TRASH) * 0x10001u;
                xrows.resize(xrows.size() + SLOTS, 0);
                rec.insert(rec.end(), rd, rd + RECDW);
                w.resize(w.size() + RECDW, -0.0f);
            }
        }
    }
    R.nrec = rec.size() / RECDW;
    R.slots = slots_total;
    R.xloads = parts_total;
    void *p = nullptr;
    so_status s = so_malloc(ctx, hdr.size() * 4, &p);
    if (s != SO_OK) return s;
    R.d_hdr = (uint32_t *)p;
    if ((s = so_malloc(ctx, rec.size() * 4, &p)) != SO_OK) return s;
    R.d_rec = (uint32_t *)p;
    if ((s = so_malloc(ctx, w.size() * 4, &p)) != SO_OK) return s;
    R.d_w = (float *)p;
    if ((s = so_malloc(ctx, xrows.size() * 4, &p)) != SO_OK) return s;
    R.d_xrows = (uint32_t *)p;
    if ((s = so_h2d(ctx, R.d_xrows, xrows.data(), xrows.size() * 4)) != SO_OK) return s;
    if ((s = so_h2d(ctx, R.d_hdr, hdr.data(), hdr.size() * 4)) != SO_OK) return s;
    if ((s = so_h2d(ctx, R.d_rec, rec.data(), rec.size() * 4)) != SO_OK) return s;
    return so_h2d(ctx, R.d_w, w.data(), w.size() * 4);
}

void so_rbmm_free(so_ellpack *E)
{
    so_rbmm &R = E->rbmm;
    if (R.d_hdr) (void)hipFree(R.d_hdr);
    if (R.d_rec) (void)hipFree(R.d_rec);
    if (R.d_w) (void)hipFree(R.d_w);
    if (R.d_xrows) (void)hipFree(R.d_xrows);
    R = so_rbmm();
}

bool so_matmul_rbm_applies(const so_ctx *ctx, const so_ellpack *E, uint32_t C)
{
    if (!(E->layouts & SO_LAYOUT_RBM) || E->rbmm.d_rec == nullptr) return false;
    if ((uint64_t)E->n * C * 4u > 0xffffffffull) return false;          // X row offsets are 32-bit byte offsets
    return (size_t)ctx->max_lds_bytes >= LDS_BYTES;
}

// Grows the context's workspace (the partial tiles of the workgroups that share a tile, a counter per tile)
// to what a launch of E with C dense columns needs.  Never while a graph is being recorded.
so_status so_matmul_rbm_reserve(so_ctx *ctx, const so_ellpack *E, uint32_t C)
{
    const so_rbmm &R = E->rbmm;
    const uint64_t tiles = (uint64_t)R.nb * so_ceil_div(C, 64);
    SO_REQUIRE(tiles * R.ksplit < (1ull << 28), "so_matmul: %u x %u output is too large for one launch", E->m, C);
    if (R.ksplit == 1) return SO_OK;
    const size_t need_part = (size_t)tiles * R.ksplit * RB * 64 * sizeof(float), need_cnt = (size_t)tiles * sizeof(uint32_t);
    if (need_part <= ctx->mm_part_bytes && need_cnt <= ctx->mm_counter_bytes) return SO_OK;
    SO_REQUIRE(!ctx->capturing, "so_matmul: the row-block-merged kernel's workspace must grow, which cannot be done while a graph is "
                                "being recorded (call so_matmul_reserve, or launch this shape once, before recording)");
    SO_HIP(hipStreamSynchronize(ctx->stream));
    if (ctx->mm_part) { (void)hipFree(ctx->mm_part); ctx->mm_part = nullptr; ctx->mm_part_bytes = 0; }
    if (ctx->mm_counters) { (void)hipFree(ctx->mm_counters); ctx->mm_counters = nullptr; ctx->mm_counter_bytes = 0; }
    const size_t pb = need_part + need_part / 4, cb = std::max<size_t>(need_cnt * 2, 4096);
    SO_HIP(hipMalloc((void **)&ctx->mm_part, pb));
    ctx->mm_part_bytes = pb;
    SO_HIP(hipMalloc((void **)&ctx->mm_counters, cb));
    ctx->mm_counter_bytes = cb;
    SO_HIP(hipMemsetAsync(ctx->mm_counters, 0, cb, ctx->stream));
    SO_HIP(hipStreamSynchronize(ctx->stream));
    return SO_OK;
}

// The records address X rows by byte offset (row * pitch): rewritten for dense width C when the handle was
// last used with another (stream-ordered; launches of one handle with different C must not overlap on
// different streams).  Never inside a recording: the rewrite would become a node of the graph, run again
// on every replay, and leave launches outside the graph with records that were never written.
so_status so_matmul_rbm_set_pitch(so_ctx *ctx, const so_ellpack *E, uint32_t C)
{
    const so_rbmm &R = E->rbmm;
    if (R.pitch == C * 4u) return SO_OK;
    SO_REQUIRE(!ctx->capturing, "so_matmul: the row-block-merged records must be rewritten for %u dense columns, which cannot be done "
                                "while a graph is being recorded (call so_matmul_reserve, or launch this shape once, before recording)", C);
    so_rbmm &Rw = const_cast<so_ellpack *>(E)->rbmm;
    const uint64_t words = R.nrec * 4;
    rbmm_offsets_kernel<<<so_ceil_div(words, 256), 256, 0, ctx->stream>>>(Rw.d_rec, Rw.d_xrows, R.nrec, C * 4u);
    Rw.pitch = C * 4u;
    return SO_OK;
}

so_status so_matmul_rbm_launch(so_ctx *ctx, const so_ellpack *E, const float *dX, uint32_t C,
                               const float *dBias, float *dY, int act)
{
    so_status rs = so_matmul_rbm_reserve(ctx, E, C);
    if (rs != SO_OK) return rs;
    if ((rs = so_matmul_rbm_set_pitch(ctx, E, C)) != SO_OK) return rs;
    switch (act) {
    case SO_ACT_RELU:    return launch_rbm<SO_ACT_RELU>(ctx, E, dX, C, dBias, dY);
    case SO_ACT_SIGMOID: return launch_rbm<SO_ACT_SIGMOID>(ctx, E, dX, C, dBias, dY);
    case SO_ACT_TANH:    return launch_rbm<SO_ACT_TANH>(ctx, E, dX, C, dBias, dY);
    default:             return launch_rbm<SO_ACT_NONE>(ctx, E, dX, C, dBias, dY);
    }
}
