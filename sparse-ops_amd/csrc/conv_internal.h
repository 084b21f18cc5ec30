// Definitions shared by the convolution translation units (conv.hip, conv_rbm.hip).
#pragma once

#include "so_internal.h"
#include "lds_sync.h"

#include <algorithm>
#include <vector>

// What the LDS-windowed kernel needs on top of the plan; built only for geometries it suits.
// The input channels are cut into chunks of `cc`; for one chunk and one tile of TH x TW output
// pixels the input window is IH x IW pixels.  A stored nonzero becomes the entry {weight bits,
// pixel offset of its tap inside the chunk's window}.  Output channels are taken `cpw` at a
// time (the channels one wave accumulates); the entries of such a channel group are one
// contiguous stream in the order the wave consumes them: chunk by chunk, inside a chunk channel
// by channel, inside a channel in slot order (slots are ordered by input channel, so a chunk is
// a slot range).  Every (chunk, channel) run is padded to a multiple of four entries with
// {-0.0, offset of an all-zero plane kept behind the window}: fma(-0, +0, acc) leaves any
// accumulator as it is.
struct so_conv_window {
    uint32_t TH = 0, TW = 0, IH = 0, IW = 0, cc = 0, nch = 0, tiles_x = 0, tiles_y = 0;
    uint32_t groups = 0;          // ceil(Cout / cpw)
    int cpw = 0;                  // output channels per wave
    uint32_t lpp = 0;             // lanes per pixel (batch tile / 4) the chunk size was chosen for: 4, 2 or 1
    int2 *d_stream = nullptr;     // all groups' streams, followed by one padding quad
    uint32_t *d_gbase = nullptr;  // [groups]: first quad (4 entries) of the group's stream
    uint32_t *d_quads = nullptr;  // [groups * nch * cpw]: quads of (group, chunk, channel in group)
};

// Record streams of the row-block-merged kernel (conv_rbm.hip) for the plan's current window layout.
struct so_conv_rbm {
    const so_rbm *src = nullptr;     // the attached format; must outlive the plan
    void *d_sets = nullptr;          // 64-byte sets of two records, all blocks, chunk after chunk
    uint32_t *d_gbase = nullptr;     // [blocks]: first set of the block's stream
    uint32_t *d_counts = nullptr;    // [blocks * chunks]: sets the loop walks for (block, chunk); 0: none
    uint64_t total_sets = 0, real_pairs = 0, slots = 0;
};

struct so_conv_plan {
    uint32_t tuned_batch = 32;   // batch the windowed layout was sized for
    uint32_t tried_lpp = 0;      // lanes per pixel of the last attempt to build the windowed layout
    so_conv_geom g;
    const so_ellpack *E = nullptr;
    int2 *d_taps = nullptr;  // per slot: x = (cin*H + dh)*W + dw (elements of B floats), y = dh<<16 | (dw & 0xffff)
    so_conv_window win;      // win.cc == 0: not built
    so_conv_rbm rbm;         // rbm.d_sets == nullptr: no streams
};

// conv_rbm.hip
void so_conv_rbm_release(so_conv_plan *plan);
so_status so_conv_rbm_rebuild(so_ctx *ctx, so_conv_plan *plan);
so_status so_conv_rbm_launch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B, const float *dBias,
                             const float *dResid, float *dY, int act, bool forced, bool *done);


constexpr int kWinThreads = 1024;
constexpr int kWinMaxPerThread = 6;   // float4 window elements a thread copies per chunk
constexpr uint32_t kWinLPP = 4;       // lanes per pixel of the preferred batch tile ...
constexpr uint32_t kWinBT = 4 * kWinLPP;   // ... of 16; batches that are only multiples of 8 or 4 use tiles of 8 or 4

// Lanes per pixel for batch B: the largest batch tile (16, 8, 4) that divides B; 0 if none does.
inline uint32_t window_lpp(uint32_t B) { return B % 16 == 0 ? 4u : B % 8 == 0 ? 2u : B % 4 == 0 ? 1u : 0u; }

struct WinArgs {
    uint32_t TH, TW, IH, IW, cc, nch, tiles_x, pg, cg, groups;
    uint32_t win_f4;    // float4 elements of one chunk's window
    uint32_t buf_f4;    // window plus the zero plane: stride between the two buffers
    uint32_t nbuf;      // 2: double-buffered windows; 1: a single chunk, nothing to overlap
    uint32_t sth, stw;  // window pixels between neighbouring output pixels
    uint32_t sbh, sbw;  // input pixels between neighbouring window pixels
    uint32_t order[16]; // slot -> output pixel of the tile (ty * TW + tx), one byte per slot; see window_pixel_order
    uint32_t mIW, mIH, mTW, mTilesX, mPg;   // window_magic of IW, IH, TW, tiles_x and pg: the kernels' index arithmetic divides by them
    so_lds::wait_status ws;   // bounded waits on the progress counters
};

// x / d for the small operands of the window index arithmetic (x * d < 2^32: window elements and
// pixels count a few thousand, the divisors are window or tile extents) as one multiply-high by
// M = ceil(2^32 / d) instead of the ~25 instructions of a general 32-bit division: exact, because
// M * d - 2^32 < d makes the error of x * M / 2^32 smaller than 1 / d.  d == 1 has no 32-bit M.
inline uint32_t window_magic(uint32_t d) { return d > 1 ? (uint32_t)(((1ull << 32) + d - 1) / d) : 0u; }
__device__ __forceinline__ uint32_t window_div(uint32_t x, uint32_t d, uint32_t M) { return d == 1u ? x : __umulhi(x, M); }

// Along an axis on which the kernel has a single tap, a strided convolution reads only every
// stride-th input pixel: the window then holds just those (one window pixel per output pixel)
// instead of all the pixels in between.
inline uint32_t window_step(uint32_t k, uint32_t stride) { return k == 1 ? 1u : stride; }
inline uint32_t window_subsample(uint32_t k, uint32_t stride) { return k == 1 ? stride : 1u; }

// Which output pixel of the tile each pixel slot of the workgroup computes (slot = lanes / lanes per
// pixel, wave after wave).  LDS serves a 16-byte read 16 lanes at a time: 16 / lpp pixels, each a run
// of 16 * lpp bytes at (window pixel index) * 16 * lpp, i.e. on the bank group (window pixel index)
// mod (16 / lpp).  Pixels taken in row-major order collide on a bank group whenever the tile's rows
// are not a multiple of 16 / lpp pixels wide (tiles 7 pixels wide: every second read takes two
// turns).  Which slot computes which pixel is free, so the slots are dealt out such that the
// pixels of each group of 16 / lpp slots fall on different bank groups wherever the tile's shape
// allows it.  At most 64 pixels per tile; the table covers all 64 slots.
inline void window_pixel_order(WinArgs &a, uint32_t lpp)
{
    const uint32_t m = 16u / lpp, npx = a.TH * a.TW;
    std::vector<std::vector<uint8_t>> bucket(m);
    for (uint32_t p = 0; p < npx && p < 64u; ++p)
        bucket[((p / a.TW) * a.sth * a.IW + (p % a.TW) * a.stw) % m].push_back((uint8_t)p);
    for (auto &b : bucket) std::reverse(b.begin(), b.end());       // pop_back hands out the lowest pixel first
    uint8_t slots[64] = {0};
    uint32_t filled = 0;
    while (filled < npx && filled < 64u) {
        // one group: a pixel from each bank group, fullest first; then, if some are exhausted, more from the fullest
        std::vector<uint32_t> by_size(m);
        for (uint32_t r = 0; r < m; ++r) by_size[r] = r;
        std::stable_sort(by_size.begin(), by_size.end(), [&](uint32_t x, uint32_t y) { return bucket[x].size() > bucket[y].size(); });
        uint32_t taken = 0;
        for (uint32_t pass = 0; taken < m && filled < npx && filled < 64u; ++pass) {
            bool any = false;
            for (uint32_t k = 0; k < m && taken < m && filled < npx && filled < 64u; ++k) {
                std::vector<uint8_t> &b = bucket[by_size[k]];
                if (b.empty()) continue;
                slots[filled++] = b.back();
                b.pop_back();
                ++taken;
                any = true;
            }
            if (!any) break;
        }
    }
    // Slots beyond the tile compute nothing but still read: they repeat an address of their own group
    // of m slots (a read that several lanes share costs the banks one turn), or the previous group's.
    for (uint32_t i = filled; i < 64u; ++i) slots[i] = (i % m != 0) ? slots[i - i % m] : (i >= m ? slots[i - m] : 0);
    for (uint32_t i = 0; i < 16; ++i)
        a.order[i] = (uint32_t)slots[4 * i] | ((uint32_t)slots[4 * i + 1] << 8) | ((uint32_t)slots[4 * i + 2] << 16) | ((uint32_t)slots[4 * i + 3] << 24);
}

// The kernels' side: the output pixel of slot `pl` (< 64).
__device__ __forceinline__ uint32_t window_slot_pixel(const WinArgs &a, uint32_t pl)
{
    uint32_t word = 0;
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) word = (pl >> 2) == i ? a.order[i] : word;
    return (word >> ((pl & 3u) * 8u)) & 0xffu;
}
