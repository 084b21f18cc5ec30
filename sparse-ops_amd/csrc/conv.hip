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
#include "conv_internal.h"
#include "dpp_steps.h"
#include "lds_sync.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

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
// entries: one 4*VEC-byte load per tap.  One batch of U taps in flight per wave.
// U = 8 when the chip is full of waves: a second batch in registers was measured
// slower (the 8 waves of a workgroup share the input window through L1 and deeper
// queues evict it).  U = 32 for launches of few waves (small batches, small
// images), where a wave's own memory-level parallelism is all the latency hiding there is.
template <int VEC, int ACT, int U>
__global__ __launch_bounds__(kChannelsPerGroup * 64)
void conv2d_implicit_kernel(const float *__restrict__ Wd, const int2 *__restrict__ taps,
                            const uint32_t *__restrict__ nnz, uint32_t r, so_conv_geom g,
                            const float *__restrict__ X, uint32_t B, uint64_t ncols,
                            const float *__restrict__ bias, const float *__restrict__ resid, float *__restrict__ Y)
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

    if constexpr (U == 32) {
        // Few waves on the chip: latency is everything.  Two register batches of 16 taps, the next
        // one issued before the current one is consumed, so tap fetch, address arithmetic, gathers
        // and multiply-adds of neighbouring batches overlap.  Branch-free taps as in the border path.
        constexpr int H = 16;
        float wa[H], wb[H], xa[H][VEC], xb[H][VEC];
        bool oka[H], okb[H];
        auto issue = [&](uint32_t j0, float (&w)[H], float (&x)[H][VEC], bool (&ok)[H]) {
            int2 t[H];
#pragma unroll
            for (int u = 0; u < H; ++u) {       // all the scalar tap loads first, as one cluster
                t[u] = trow[j0 + u];
                w[u] = wrow[j0 + u];
            }
#pragma unroll
            for (int u = 0; u < H; ++u) {
                const int32_t hin = h0 + (t[u].y >> 16), win = w0 + (int32_t)(int16_t)(t[u].y & 0xffff);
                ok[u] = ((uint32_t)hin < g.H_in) & ((uint32_t)win < g.W_in);      // '&': no branch per tap
                const int64_t off = lanebase + (int64_t)t[u].x * (int64_t)B;
                conv_load<VEC>(X + (ok[u] ? off : (int64_t)b), x[u]);
            }
        };
        auto consume = [&](const float (&w)[H], const float (&x)[H][VEC], const bool (&ok)[H]) {
#pragma unroll
            for (int u = 0; u < H; ++u)
#pragma unroll
                for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(w[u], ok[u] ? x[u][v] : 0.0f, acc[v]);
        };
        const uint32_t nb = cnt / H;
        if (nb) issue(0, wa, xa, oka);
        uint32_t bi = 0;
        for (; bi + 1 < nb; bi += 2) {
            issue((bi + 1) * H, wb, xb, okb);
            consume(wa, xa, oka);
            if (bi + 2 < nb) issue((bi + 2) * H, wa, xa, oka);
            consume(wb, xb, okb);
        }
        if (nb & 1u) consume(wa, xa, oka);
        // the partial last batch in one round trip: slots past the end re-read the last tap and are
        // dropped by a wave-uniform test
        if (const uint32_t rem = cnt - nb * H) {
            const uint32_t j0 = nb * H;
            int2 t[H];
#pragma unroll
            for (int u = 0; u < H; ++u) {
                const uint32_t j = j0 + min((uint32_t)u, rem - 1u);
                t[u] = trow[j];
                wa[u] = wrow[j];
            }
#pragma unroll
            for (int u = 0; u < H; ++u) {
                const int32_t hin = h0 + (t[u].y >> 16), win = w0 + (int32_t)(int16_t)(t[u].y & 0xffff);
                oka[u] = ((uint32_t)hin < g.H_in) & ((uint32_t)win < g.W_in);
                const int64_t off = lanebase + (int64_t)t[u].x * (int64_t)B;
                conv_load<VEC>(X + (oka[u] ? off : (int64_t)b), xa[u]);
            }
#pragma unroll
            for (int u = 0; u < H; ++u)
                if ((uint32_t)u < rem) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = __builtin_fmaf(wa[u], oka[u] ? xa[u][v] : 0.0f, acc[v]);
                }
        }
    } else if (__all(interior)) {
        const float *__restrict__ xl = X + lanebase;
        uint32_t j = 0;
        for (; j + U <= cnt; j += U) {
            float w[U], x[U][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                w[u] = wrow[j + u];
                conv_load<VEC>(xl + (int64_t)trow[j + u].x * (int64_t)B, x[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
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
        for (; j + U <= cnt; j += U) {
            float w[U], x[U][VEC];
            bool ok[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int2 t = trow[j + u];
                w[u] = wrow[j + u];
                const int32_t hin = h0 + (t.y >> 16), win = w0 + (int32_t)(int16_t)(t.y & 0xffff);
                ok[u] = (uint32_t)hin < g.H_in && (uint32_t)win < g.W_in;
                conv_load<VEC>(ok[u] ? X + lanebase + (int64_t)t.x * (int64_t)B : xsafe, x[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
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
        if (resid) {                     // the residual Add that follows the convolution: conv + skip, then the activation
            float rv[VEC];
            conv_load<VEC>(resid + (size_t)co * ncols + q, rv);
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] += rv[v];
        }
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


// ---- LDS-windowed variant -------------------------------------------------------------
//
// A workgroup of 16 waves owns a tile of TH x TW output pixels x BT batch entries and a block
// of output channels.  It walks the input channels in chunks; a chunk's input window (halo
// included, out-of-image pixels as zeros) is copied to LDS once and every tap of every output
// channel of the block is then a 16-byte LDS read, which LDS delivers at more than twice the
// rate the L1 gathers of the kernel above sustain.  Lanes: LPP = BT/4 lanes per pixel (4 batch
// entries each), so a wave covers 64/LPP pixels; the 16 waves are PG pixel groups x CG channel
// groups and a wave accumulates CPW output channels.  The batch tile is 16 (LPP = 4): measured
// against 32 and 8 it was the fastest on every layer of the ResNet-18-shaped stack, because the
// smaller window lets a chunk hold twice the channels (longer runs per channel, half the barriers).  Entries are wave-uniform.  With
// 8 or 4 channels per wave they arrive through scalar loads, four at a time and one quad ahead, so
// the weight is a scalar operand of the multiply-adds and the tap offset a scalar addend of the
// LDS address; with fewer channels per wave (fewer, longer runs and usually fewer waves to hide
// a scalar load behind) they are held one per lane and handed round by DPP (dpp_steps.h), 16
// entries per vector load, one group ahead.  Per output the
// multiply-adds run in slot order (chunks ascend, slots ascend inside a chunk): same bits as
// the kernel above.  Windows are double-buffered: chunk t+1 is fetched into registers while
// chunk t is computed.
// Brings the cache lines of `quads` stream quads (32 bytes each) from `p` on into the scalar
// cache: one scalar load per 64-byte line, all in flight together, then one wait.  LDS reads and
// scalar loads share one counter and scalar loads return out of order, so every wait for LDS data
// in the step loop also waits for the scalar load in flight; touched ahead, once per chunk, those
// loads hit (measured: 56x56x64 layer at batch 32 from 67 to 63 us).
__device__ __forceinline__ void touch_stream(const int4 *p, uint32_t quads, uint32_t part, uint32_t parts)
{
    // the lines of the range in groups of four (up to three lines past its end: the stream ends with
    // padding); the waves that walk the same stream -- the pixel groups of a channel group -- take
    // every parts-th group each
    uint32_t groups = ((quads * 32u + 32u + 63u) / 64u + 3u) / 4u, sink;      // p may sit in the middle of a line
    if (groups <= part) return;
    groups = (groups - part + parts - 1u) / parts;
    p += 16u * part;
    const uint32_t stride = 256u * parts;
    asm volatile(
        "L_touch_%=:\n\t"
        "s_load_dword %[d], s[34:35], 0x0\n\t"
        "s_load_dword %[d], s[34:35], 0x40\n\t"
        "s_load_dword %[d], s[34:35], 0x80\n\t"
        "s_load_dword %[d], s[34:35], 0xc0\n\t"
        "s_add_u32 s34, s34, %[st]\n\t"
        "s_addc_u32 s35, s35, 0\n\t"
        "s_sub_u32 %[n], %[n], 1\n\t"
        "s_cmp_lg_u32 %[n], 0\n\t"
        "s_cbranch_scc1 L_touch_%=\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        : [d] "=&s"(sink), "+{s[34:35]}"(p), [n] "+s"(groups)
        : [st] "s"(stride)
        : "scc");
}

// The four waves that share a SIMD are served oldest first: left alone, the first of them finishes a
// chunk's steps in half the time of the last (measured with the shader clock on the 56x56x64 layer:
// 14.1 k, 17.4 k, 22.1 k, 28.7 k clocks by age), and everybody then waits for the last one at the
// chunk's barrier with the SIMD mostly idle.  Each wave therefore keeps taking a new priority, the
// four of a SIMD four different ones at the same point of their work (wave / 4 is the wave's age rank
// on its SIMD).  Measured at batch 32: 56x56x64 layer 63.1 -> 58.5 us, 28x28x128 67.3 -> 65.1,
// 14x14x256 60.2 -> 58.4; inside the 8-channel form's quad loop the extra branch costs what it gains.
__device__ __forceinline__ void rotate_priority(uint32_t turn)
{
    switch (turn & 3u) {
    case 0: __builtin_amdgcn_s_setprio(0); break;
    case 1: __builtin_amdgcn_s_setprio(1); break;
    case 2: __builtin_amdgcn_s_setprio(2); break;
    default: __builtin_amdgcn_s_setprio(3); break;
    }
}

template <int CPW, int LPP, int ACT>
__global__ __launch_bounds__(kWinThreads)
void conv2d_window_kernel(const int4 *__restrict__ stream, const uint32_t *__restrict__ gbase,
                          const uint32_t *__restrict__ quads, WinArgs a, so_conv_geom g,
                          const float *__restrict__ X, uint32_t B, const float *__restrict__ bias,
                          const float *__restrict__ resid, float *__restrict__ Y)
{
    extern __shared__ float4 win_lds[];
    constexpr uint32_t BT = LPP * 4, PPW = 64 / LPP, SHIFT = (LPP == 8 ? 7 : LPP == 4 ? 6 : LPP == 2 ? 5 : 4);
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t cgi = window_div(wave, a.pg, a.mPg), pgi = wave - cgi * a.pg;
    const uint32_t tile_y = window_div(blockIdx.x, a.tiles_x, a.mTilesX);
    const uint32_t th0 = tile_y * a.TH, tw0 = (blockIdx.x - tile_y * a.tiles_x) * a.TW;
    const uint32_t grp = blockIdx.y * a.cg + cgi;                    // channel group of this wave
    const uint32_t co0 = grp * CPW;
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
    int32_t goff[kWinMaxPerThread];      // float offset from the chunk's first channel; -1: outside the image
    uint32_t gcl[kWinMaxPerThread];      // channel inside the chunk; 0xffffffff: no such element
#pragma unroll
    for (int k = 0; k < kWinMaxPerThread; ++k) {
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

    float4 xr[kWinMaxPerThread];
    auto fetch_window = [&](uint32_t t) {
        const float *__restrict__ Xc = X + (size_t)t * chunk_floats;
        const uint32_t cleft = g.Cin - t * a.cc;                       // channels left from this chunk on
#pragma unroll
        for (int k = 0; k < kWinMaxPerThread; ++k) {
            xr[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (goff[k] >= 0 && gcl[k] < cleft) xr[k] = *reinterpret_cast<const float4 *>(Xc + goff[k]);
        }
    };
    auto store_window = [&](uint32_t buf) {
#pragma unroll
        for (int k = 0; k < kWinMaxPerThread; ++k)
            if (gcl[k] != 0xffffffffu) win_lds[buf * a.buf_f4 + tid + (uint32_t)k * kWinThreads] = xr[k];
    };

    float acc[CPW][4];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        const float b0 = (bias && computes && co0 + c < g.Cout) ? bias[co0 + c] : 0.0f;
        acc[c][0] = acc[c][1] = acc[c][2] = acc[c][3] = b0;
    }

    // the all-zero plane behind each window buffer (padding entries point into it)
    for (uint32_t i = tid; i < a.buf_f4 - a.win_f4; i += kWinThreads) {
        win_lds[a.win_f4 + i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (a.nbuf == 2) win_lds[a.buf_f4 + a.win_f4 + i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    // progress counters behind the buffers: [0], [1] windows stored into buffer 0 / 1 (x 16 waves), [2], [3] chunks read out of them
    const uint32_t sync_base = so_lds::lds_address(win_lds + (size_t)a.nbuf * a.buf_f4);
    if (a.nbuf == 2 && tid < 4) reinterpret_cast<uint32_t *>(win_lds + (size_t)a.nbuf * a.buf_f4)[tid] = tid == 0 ? 16u : 0u;
    fetch_window(0);                  // stored below, once the entry stream is set up: the two latencies overlap

    // The wave's entry stream: one quad = 4 entries = two int4 {w0, o0, w1, o1}, {w2, o2, w3, o3}.
    // `cur` is the quad about to be used, the next one is requested before cur is consumed; the
    // stream ends with a padding quad, so the request after the last quad is harmless.
    // (read through the constant address space: that keeps them scalar loads next to the inline
    // assembly of touch_stream)
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef const i32x4 __attribute__((address_space(4))) *const_stream;
    const int4 *__restrict__ sp0 = stream + 2 * (size_t)gbase[gi];
    const_stream sp = (const_stream)(uintptr_t)sp0;
    const uint32_t *__restrict__ qp = quads + (size_t)gi * a.nch * CPW;
    i32x4 cur0 = {0, 0, 0, 0}, cur1 = cur0;
    // LANE_ENT: the entries sit in lanes instead (lane l of every 16-lane row holds entry l of the
    // next 16), fetched with vector loads one group ahead and broadcast by DPP: vector loads have
    // their own counter, so waiting for LDS data never waits for entries.  A DPP multiply-add keeps
    // the vector unit busy a third longer than one with a scalar weight, though, so the scalar form
    // wins wherever a wave has enough runs per chunk to amortise its scalar loads: measured on the
    // ResNet-18-shaped layers at batch 32, scalar against lanes: 8 channels per wave 55 against 60 us,
    // 4 channels 56.1 against 63.2, 2 channels 58.8 against 56.6; small batches use 1-2 channels.
    constexpr bool LANE_ENT = CPW < 4;
    // priorities rotate on the full batch tile only: on the smaller ones (batches below 16) it measured 5 % slower
    constexpr bool ROTATE = LPP == 4;
    // progress counters instead of a barrier per chunk: the same (batch 8: 0.466 -> 0.474 ms, batch 1: 0.365 -> 0.374 with them)
    constexpr bool DRIFT = LPP == 4;
    const int2 *__restrict__ ep = reinterpret_cast<const int2 *>(sp0) + (lane & 15u);
    int2 ecur = make_int2(0, 0);
    uint32_t qtouch = 0;                                             // quads of the chunk about to start
    if constexpr (LANE_ENT) {
        ecur = ep[0];
    } else {
        if (computes) {
#pragma unroll
            for (int c = 0; c < CPW; ++c) qtouch += qp[c];
        }
        touch_stream(sp0, qtouch + 1u, pgi, a.pg);
        cur0 = sp[0];
        cur1 = sp[1];
        sp += 2;
    }
    store_window(0);
    __syncthreads();

    const char *lds_bytes = reinterpret_cast<const char *>(win_lds);
    for (uint32_t t = 0; t < a.nch; ++t) {
        const bool more = t + 1 < a.nch;
        if (more) fetch_window(t + 1);
        const uint32_t cur_buf = a.nbuf == 2 ? (t & 1u) : 0u;
        const uint32_t base = lanebase + cur_buf * buf_bytes;
        uint32_t nq[CPW];
#pragma unroll
        for (int c = 0; c < CPW; ++c) nq[c] = computes ? qp[t * CPW + c] : 0u;
        // Half-way through the chunk the wave stores its part of the next window, as soon as every wave
        // has finished the chunk before this one (which read the buffer it goes to).  A wave that is
        // done with its steps then only needs every wave to be past that half-way point, not to be
        // done as well: the waves of a SIMD finish a chunk up to a third of its length apart.
        bool stored = !(DRIFT && more && a.nbuf == 2);
        auto store_next = [&]() {
            if (stored) return;
            stored = true;
            so_lds::wait(sync_base + 8u + ((t + 1u) & 1u) * 4u, 16u * ((t + 1u) / 2u), a.ws);
            store_window((t + 1u) & 1u);
            so_lds::signal(sync_base + ((t + 1u) & 1u) * 4u, lane);
        };
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
            if (CPW >= 2 && c == CPW / 2) store_next();
            const uint32_t turn = (wave >> 2) + (uint32_t)c + t;      // a new priority per run; per group of 16 entries where the entries sit in lanes
            if constexpr (ROTATE) rotate_priority(turn);
            if constexpr (LANE_ENT && CPW <= 2) {
                // Pipelined: a quad's LDS reads overlap the previous quad's multiply-adds all through
                // the run (so_dpp::group16).  Measured on ResNet-18 shapes at batch 32: 14x14x256
                // (2 channels per wave) 63.5 -> 58.4 us, 7x7x512 (1 per wave) 69.1 -> 66.1 us; with 4
                // channels per wave the four copies of these bodies made 28x28x128 11 % slower.
                const uint32_t n = nq[c];
                const char *xb = lds_bytes + base;
                float4 xA[4], xB[4];
                if (n >= 4u) {
                    ep += 16;
                    int2 enxt = ep[0];                                    // the stream ends with 16 padding entries
                    so_dpp::group16<false>(xb, __int_as_float(ecur.x), (uint32_t)ecur.y << SHIFT, 0.0f, xA, xB, acc[c]);
                    float ewp = __int_as_float(ecur.x);
                    ecur = enxt;
                    uint32_t q = 4u;
                    const uint32_t q_mid = CPW == 1 ? n / 8u * 4u : 0xffffffffu;
                    for (; q + 4u <= n; q += 4u) {
                        if (CPW == 1 && q == q_mid) store_next();
                        if constexpr (ROTATE) rotate_priority(turn + (q >> 2));
                        ep += 16;
                        enxt = ep[0];
                        so_dpp::group16<true>(xb, __int_as_float(ecur.x), (uint32_t)ecur.y << SHIFT, ewp, xA, xB, acc[c]);
                        ewp = __int_as_float(ecur.x);
                        ecur = enxt;
                    }
                    if (q < n) {
                        ep += 4u * (n - q);
                        enxt = ep[0];
                        so_dpp::group_tail<true>(n - q, xb, __int_as_float(ecur.x), (uint32_t)ecur.y << SHIFT, ewp, xA, xB, acc[c]);
                        ecur = enxt;
                    } else {
                        so_dpp::group_drain(ewp, xB, acc[c]);
                    }
                } else if (n != 0u) {
                    ep += 4u * n;
                    const int2 enxt = ep[0];
                    so_dpp::group_tail<false>(n, xb, __int_as_float(ecur.x), (uint32_t)ecur.y << SHIFT, 0.0f, xA, xB, acc[c]);
                    ecur = enxt;
                }
                continue;
            }
            if constexpr (LANE_ENT) {
                for (uint32_t q = 0; q < nq[c]; q += 4u) {
                    if (ROTATE && q) rotate_priority(turn + (q >> 2));
                    const uint32_t steps = 4u * min(4u, nq[c] - q);      // this group: 4, 8, 12 or 16 entries
                    ep += steps;
                    const int2 enxt = ep[0];                              // the stream ends with 16 padding entries
                    so_dpp::tiled_chunk(lds_bytes + base, __int_as_float(ecur.x), (uint32_t)ecur.y << SHIFT, steps, acc[c]);
                    ecur = enxt;
                }
                continue;
            }
            for (uint32_t q = 0; q < nq[c]; ++q) {
                const i32x4 nxt0 = sp[0], nxt1 = sp[1];
                sp += 2;
                const float4 x0 = *reinterpret_cast<const float4 *>(lds_bytes + base + ((uint32_t)cur0.y << SHIFT));
                const float4 x1 = *reinterpret_cast<const float4 *>(lds_bytes + base + ((uint32_t)cur0.w << SHIFT));
                const float4 x2 = *reinterpret_cast<const float4 *>(lds_bytes + base + ((uint32_t)cur1.y << SHIFT));
                const float4 x3 = *reinterpret_cast<const float4 *>(lds_bytes + base + ((uint32_t)cur1.w << SHIFT));
                const float w0 = __int_as_float(cur0.x), w1 = __int_as_float(cur0.z);
                const float w2 = __int_as_float(cur1.x), w3 = __int_as_float(cur1.z);
                acc[c][0] = __builtin_fmaf(w0, x0.x, acc[c][0]); acc[c][1] = __builtin_fmaf(w0, x0.y, acc[c][1]);
                acc[c][2] = __builtin_fmaf(w0, x0.z, acc[c][2]); acc[c][3] = __builtin_fmaf(w0, x0.w, acc[c][3]);
                acc[c][0] = __builtin_fmaf(w1, x1.x, acc[c][0]); acc[c][1] = __builtin_fmaf(w1, x1.y, acc[c][1]);
                acc[c][2] = __builtin_fmaf(w1, x1.z, acc[c][2]); acc[c][3] = __builtin_fmaf(w1, x1.w, acc[c][3]);
                acc[c][0] = __builtin_fmaf(w2, x2.x, acc[c][0]); acc[c][1] = __builtin_fmaf(w2, x2.y, acc[c][1]);
                acc[c][2] = __builtin_fmaf(w2, x2.z, acc[c][2]); acc[c][3] = __builtin_fmaf(w2, x2.w, acc[c][3]);
                acc[c][0] = __builtin_fmaf(w3, x3.x, acc[c][0]); acc[c][1] = __builtin_fmaf(w3, x3.y, acc[c][1]);
                acc[c][2] = __builtin_fmaf(w3, x3.z, acc[c][2]); acc[c][3] = __builtin_fmaf(w3, x3.w, acc[c][3]);
                cur0 = nxt0;
                cur1 = nxt1;
            }
        }
        if constexpr (!LANE_ENT) {
            if (more && computes) {                // the next chunk's entries, while the slower waves finish this one
                uint32_t qn = 0;
#pragma unroll
                for (int c = 0; c < CPW; ++c) qn += qp[(t + 1) * CPW + c];
                if (qn) touch_stream((const int4 *)(uintptr_t)sp, qn, pgi, a.pg);
            }
        }
        if (DRIFT && a.nbuf == 2) {
            store_next();
            so_lds::signal(sync_base + 8u + cur_buf * 4u, lane);                    // done reading this chunk's buffer
            if (more) so_lds::wait(sync_base + (cur_buf ^ 1u) * 4u, 16u * ((t + 1u) / 2u + 1u), a.ws);   // the next window is complete
        } else if (a.nbuf == 2) {
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
        for (int c = 0; c < CPW; ++c) {
            const uint32_t co = co0 + c;
            if (co < g.Cout) {
                const size_t at = (((size_t)co * g.H_out + ho) * g.W_out + wo) * B + bz + b4 * 4u;
                if (resid) {             // conv + skip, then the activation
                    const float4 rv = *reinterpret_cast<const float4 *>(resid + at);
                    acc[c][0] += rv.x; acc[c][1] += rv.y; acc[c][2] += rv.z; acc[c][3] += rv.w;
                }
                float4 out;
                out.x = so_epilogue<ACT>(acc[c][0]); out.y = so_epilogue<ACT>(acc[c][1]);
                out.z = so_epilogue<ACT>(acc[c][2]); out.w = so_epilogue<ACT>(acc[c][3]);
                *reinterpret_cast<float4 *>(Y + at) = out;
            }
        }
    }
}

template <int CPW, int LPP>
void window_launch_act(so_ctx *ctx, const so_conv_plan *plan, const WinArgs &a, dim3 grid, size_t lds,
                       const float *dX, uint32_t B, const float *dBias, const float *dResid, float *dY, int act)
{
#define SO_WIN_LAUNCH(A)                                                                                   \
    conv2d_window_kernel<CPW, LPP, A><<<grid, kWinThreads, lds, ctx->stream>>>(                            \
        reinterpret_cast<const int4 *>(plan->win.d_stream), plan->win.d_gbase, plan->win.d_quads, a,       \
        plan->g, dX, B, dBias, dResid, dY)
    switch (act) {
    case SO_ACT_RELU:    SO_WIN_LAUNCH(SO_ACT_RELU); break;
    case SO_ACT_SIGMOID: SO_WIN_LAUNCH(SO_ACT_SIGMOID); break;
    case SO_ACT_TANH:    SO_WIN_LAUNCH(SO_ACT_TANH); break;
    default:             SO_WIN_LAUNCH(SO_ACT_NONE); break;
    }
#undef SO_WIN_LAUNCH
}

// The windowed kernels use more than the default 64 KB of dynamic LDS: raise the limit of every
// instantiation once, at plan creation (never from so_conv2d, which may run under graph capture).
template <int CPW, int LPP>
hipError_t window_allow_lds(so_ctx *ctx)
{
    hipError_t e = hipSuccess;
    const void *k[4] = {(const void *)conv2d_window_kernel<CPW, LPP, SO_ACT_NONE>, (const void *)conv2d_window_kernel<CPW, LPP, SO_ACT_RELU>,
                        (const void *)conv2d_window_kernel<CPW, LPP, SO_ACT_SIGMOID>, (const void *)conv2d_window_kernel<CPW, LPP, SO_ACT_TANH>};
    for (const void *f : k)
        if (e == hipSuccess) e = so_allow_big_lds(ctx, f);
    return e;
}

so_status window_configure(so_ctx *ctx)
{
    SO_HIP((window_allow_lds<8, 4>(ctx))); SO_HIP((window_allow_lds<4, 4>(ctx)));
    SO_HIP((window_allow_lds<2, 4>(ctx))); SO_HIP((window_allow_lds<1, 4>(ctx)));
    SO_HIP((window_allow_lds<8, 2>(ctx))); SO_HIP((window_allow_lds<4, 2>(ctx)));
    SO_HIP((window_allow_lds<2, 2>(ctx))); SO_HIP((window_allow_lds<1, 2>(ctx)));
    SO_HIP((window_allow_lds<8, 1>(ctx))); SO_HIP((window_allow_lds<4, 1>(ctx)));
    SO_HIP((window_allow_lds<2, 1>(ctx))); SO_HIP((window_allow_lds<1, 1>(ctx)));
    return SO_OK;
}

// Workgroups the windowed kernel launches for batch B with `cpw` channels per wave.
uint64_t window_workgroups(const so_conv_window &w, uint32_t cout, uint32_t cpw, uint32_t B)
{
    const uint32_t lpp = std::max(1u, window_lpp(B));
    const uint32_t pg = so_ceil_div(w.TH * w.TW, 64u / lpp), cg = 16u / pg;
    return (uint64_t)w.tiles_x * w.tiles_y * so_ceil_div(so_ceil_div(cout, cpw), cg) * std::max(1u, B / (4u * lpp));
}

// Launches the windowed kernel if the plan has the layout, the batch suits it and the grid
// covers the chip; *done says whether it did.
template <uint32_t LPP>
so_status window_launch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B, const float *dBias,
                        const float *dResid, float *dY, int act, bool forced, bool *done)
{
    const so_conv_window &w = plan->win;
    constexpr uint32_t PPW = 64 / LPP;
    WinArgs a;
    a.TH = w.TH; a.TW = w.TW; a.IH = w.IH; a.IW = w.IW; a.cc = w.cc; a.nch = w.nch; a.tiles_x = w.tiles_x;
    a.groups = w.groups;
    a.pg = so_ceil_div(w.TH * w.TW, PPW);
    a.cg = 16 / a.pg;
    // A grid of at most half the CUs (small batches on small images): halve the computing waves of
    // a workgroup -- the others still help copying the window -- while the doubled grid still fits
    // the chip at one workgroup per CU.  The waves of a CU share its LDS read rate, so the layer's
    // steps then run on twice the CUs (7x7x512 layer at batch 1: 54.5 -> 37.7 us).  Where the grid
    // already covers more than half the chip this loses (the workgroups no longer fit one round).
    {
        const uint64_t spatial = (uint64_t)w.tiles_x * w.tiles_y * (B / (4 * LPP));
        const uint32_t floor_cg = ctx->tune.conv_min_cg > 0 ? (uint32_t)ctx->tune.conv_min_cg : 1u;
        while (a.cg > floor_cg && a.cg % 2 == 0 && spatial * so_ceil_div(w.groups, a.cg) <= (uint64_t)ctx->compute_units / 2) a.cg /= 2;
    }
    a.win_f4 = w.cc * w.IH * w.IW * LPP;
    a.buf_f4 = (w.cc + 1) * w.IH * w.IW * LPP;
    a.nbuf = w.nch > 1 ? 2u : 1u;
    a.sth = window_step(plan->g.kH, plan->g.stride_h); a.stw = window_step(plan->g.kW, plan->g.stride_w);
    a.sbh = window_subsample(plan->g.kH, plan->g.stride_h); a.sbw = window_subsample(plan->g.kW, plan->g.stride_w);
    window_pixel_order(a, LPP);
    a.mIW = window_magic(a.IW); a.mIH = window_magic(a.IH); a.mTW = window_magic(a.TW);
    a.mTilesX = window_magic(a.tiles_x); a.mPg = window_magic(a.pg);
    a.ws = so_lds::wait_status{ctx->tune.wait_spins >= 0 ? (uint32_t)ctx->tune.wait_spins : so_lds::kSyncSpins, ctx->d_wait_gave_up};
    const size_t lds = (size_t)a.nbuf * a.buf_f4 * 16 + so_lds::kSyncBytes;
    // a layout whose chunks were sized for a smaller batch tile than this batch's does not fit
    if (LPP > w.lpp && (lds > (size_t)ctx->max_lds_bytes || a.win_f4 > (uint32_t)kWinMaxPerThread * kWinThreads)) return SO_OK;
    const dim3 grid(w.tiles_x * w.tiles_y, so_ceil_div(w.groups, a.cg), B / (4 * LPP));
    const uint64_t wgs = (uint64_t)grid.x * grid.y * grid.z;
    // Even a grid that covers an eighth of the chip beats the gather kernel on long rows (measured on the
    // 14x14 and 7x7 layers of a ResNet-18-shaped stack at batch 8); below that the gather kernel's finer waves win.
    if (!forced && 8 * wgs < (uint64_t)ctx->compute_units) return SO_OK;
    if (grid.y > 65535u || grid.z > 65535u) return SO_OK;
    switch (w.cpw) {
    case 8:  window_launch_act<8, (int)LPP>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    case 4:  window_launch_act<4, (int)LPP>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    case 2:  window_launch_act<2, (int)LPP>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    default: window_launch_act<1, (int)LPP>(ctx, plan, a, grid, lds, dX, B, dBias, dResid, dY, act); break;
    }
    ctx->waits_pending = true;
    *done = true;
    return SO_OK;
}

template <int VEC>
void conv_launch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B, uint64_t ncols,
                 const float *dBias, const float *dResid, float *dY, int act)
{
    const so_conv_geom &g = plan->g;
    const so_ellpack *E = plan->E;
    const dim3 grid((uint32_t)((ncols + 64ull * VEC - 1) / (64ull * VEC)), so_ceil_div(g.Cout, kChannelsPerGroup));
    // at most 2 waves per SIMD in the whole launch and rows long enough for its batches
    const bool few = (uint64_t)grid.x * g.Cout <= 8ull * (uint64_t)ctx->compute_units && E->max_nnz >= 64;
#define SO_CONV_LAUNCH(A)                                                                          \
    do {                                                                                           \
        if (few)                                                                                   \
            conv2d_implicit_kernel<VEC, A, 32><<<grid, kChannelsPerGroup * 64, 0, ctx->stream>>>(  \
                E->d_Wd, plan->d_taps, E->d_nnz, E->r, g, dX, B, ncols, dBias, dResid, dY);        \
        else                                                                                       \
            conv2d_implicit_kernel<VEC, A, 8><<<grid, kChannelsPerGroup * 64, 0, ctx->stream>>>(   \
                E->d_Wd, plan->d_taps, E->d_nnz, E->r, g, dX, B, ncols, dBias, dResid, dY);        \
    } while (0)
    switch (act) {
    case SO_ACT_RELU:    SO_CONV_LAUNCH(SO_ACT_RELU); break;
    case SO_ACT_SIGMOID: SO_CONV_LAUNCH(SO_ACT_SIGMOID); break;
    case SO_ACT_TANH:    SO_CONV_LAUNCH(SO_ACT_TANH); break;
    default:             SO_CONV_LAUNCH(SO_ACT_NONE); break;
    }
#undef SO_CONV_LAUNCH
}


// Channels per wave for batch `batch`.  Cost of a layer ~ rounds of workgroups over the chip x
// channels per wave x (fixed + per-wave share of the chunk overhead + per-run overhead), `run`
// being the mean number of nonzeros per (channel, chunk); constants fitted on MI355X to the 3x3
// layers of a ResNet-18-shaped stack at batch 32.
int choose_cpw(const so_ctx *ctx, const so_conv_window &w, uint32_t cout, double run, uint32_t batch)
{
    int best = 1, cpw_max = 8;
    if (ctx->tune.conv_cpw > 0) cpw_max = ctx->tune.conv_cpw;
    double best_cost = 0.0;
    for (int cpw : {8, 4, 2, 1}) {
        if (cpw > cpw_max && cpw != 1) continue;
        const uint64_t wgs = window_workgroups(w, cout, (uint32_t)cpw, batch);
        const double rounds = (double)so_ceil_div((uint32_t)std::min<uint64_t>(wgs, 1u << 30), (uint32_t)ctx->compute_units);
        const double cost = rounds * cpw * (6.5 + 10.0 / cpw + 29.0 / run);
        if (best_cost == 0.0 || cost < best_cost) { best_cost = cost; best = cpw; }
    }
    return best;
}

// Chooses tile, channel chunk and channels per wave for the windowed kernel and uploads its
// arrays.  Leaves plan->win.cc == 0 when the geometry does not suit the kernel (a chunk must
// hold enough nonzeros to amortise its copy and barrier; the whole output must give the chip
// enough workgroups at batch tile 32).
so_status build_window(so_ctx *ctx, so_conv_plan *plan, const std::vector<uint32_t> &idx,
                       const std::vector<uint32_t> &nnz, const std::vector<float> &Wd, uint32_t batch)
{
    const so_conv_geom &g = plan->g;
    const so_ellpack *E = plan->E;
    const uint32_t kHW = g.kH * g.kW;
    plan->tried_lpp = window_lpp(batch) ? window_lpp(batch) : kWinLPP;
    if (kHW == 0 || E->r == 0 || E->total_nnz == 0) return SO_OK;
    if (!E->ascending) return SO_OK;     // a chunk of input channels must be a slot range of every row
    // Tile: fewest tiles, then smallest window.
    uint32_t bestTH = 0, bestTW = 0;
    uint64_t best_tiles = ~0ull, best_win = ~0ull;
    // At most 32 output pixels per tile; 16 for small images (up to 16 x 16 output pixels), where the
    // smaller window lets a chunk hold more channels and the extra tiles give the chip more workgroups
    // (measured: 14 x 14 layer 79 -> 71 us, 7 x 7 layer 89 -> 81 us; 28 x 28 and 56 x 56 lose 8-25 %).
    // Those sizes are for the batch tile of 16 (4 lanes per pixel).  A batch tile of 8 or 4 puts 2 or
    // 4 times the pixels on a wave's 64 lanes and in the same LDS: the tile is then one wave of
    // pixels, 32 or 64 (measured on the stack at batch 1: 0.478 -> 0.416 ms; at batch 8: 0.549 -> 0.523).
    const uint32_t lpp_for_batch = window_lpp(batch) ? window_lpp(batch) : kWinLPP;
    uint32_t max_px = (uint64_t)g.H_out * g.W_out <= 256 ? 16u : 32u;
    if (lpp_for_batch < kWinLPP) max_px = 64u / lpp_for_batch;
    if (ctx->tune.conv_tilepx > 0) max_px = std::min(64u, (uint32_t)ctx->tune.conv_tilepx);   // the slot table holds 64 pixels
    for (uint32_t th = 1; th <= max_px && th <= g.H_out; ++th)
        for (uint32_t tw = 1; th * tw <= max_px && tw <= g.W_out; ++tw) {
            const uint64_t tiles = (uint64_t)so_ceil_div(g.H_out, th) * so_ceil_div(g.W_out, tw);
            const uint64_t win = (uint64_t)((th - 1) * window_step(g.kH, g.stride_h) + (g.kH - 1) * g.dil_h + 1) *
                                 ((tw - 1) * window_step(g.kW, g.stride_w) + (g.kW - 1) * g.dil_w + 1);
            if (tiles < best_tiles || (tiles == best_tiles && win < best_win)) {
                best_tiles = tiles; best_win = win; bestTH = th; bestTW = tw;
            }
        }
    if (bestTH == 0) return SO_OK;
    so_conv_window w;
    w.TH = bestTH; w.TW = bestTW;
    w.IH = (w.TH - 1) * window_step(g.kH, g.stride_h) + (g.kH - 1) * g.dil_h + 1;
    w.IW = (w.TW - 1) * window_step(g.kW, g.stride_w) + (g.kW - 1) * g.dil_w + 1;
    w.tiles_y = so_ceil_div(g.H_out, w.TH);
    w.tiles_x = so_ceil_div(g.W_out, w.TW);
    if ((uint64_t)w.IH * w.IW > 4096) return SO_OK;
    // the kernels turn a workgroup's index into its tile with window_div: index * tiles_x must fit 32 bits
    if ((uint64_t)w.tiles_x * w.tiles_x * w.tiles_y >= (1ull << 32)) return SO_OK;
    // Channel chunk: two windows (plus their zero planes) fit LDS, one window fits the copy loop.
    // Both depend on the batch tile (16, 8 or 4 entries): a smaller tile lets a chunk hold more
    // channels, i.e. fewer chunks, fewer barriers and longer runs -- what small batches, whose
    // launches are bound by latency, need.  A layout sized for a batch tile also serves smaller ones.
    w.lpp = lpp_for_batch;
    const uint64_t px_bytes = w.lpp * 16, lds_budget = (uint64_t)ctx->max_lds_bytes - so_lds::kSyncBytes;     // room for the progress counters
    uint32_t cc = g.Cin;
    while (cc > 0 && ((cc < g.Cin ? 2ull : 1ull) * (cc + 1) * w.IH * w.IW * px_bytes > lds_budget ||
                      (uint64_t)cc * w.IH * w.IW * w.lpp > (uint64_t)kWinMaxPerThread * kWinThreads))
        --cc;
    if (cc == 0) return SO_OK;
    w.nch = so_ceil_div(g.Cin, cc);
    cc = so_ceil_div(g.Cin, w.nch);                 // same number of chunks, evenly filled
    w.cc = cc;
    // Enough nonzeros per (channel, chunk) to pay for the chunk's barrier and copy.
    const double nnz_avg = (double)E->total_nnz / (double)g.Cout;
    const double run = nnz_avg / w.nch;
    if (run < 6.0) return SO_OK;
    if ((uint64_t)cc * g.H_in * g.W_in >= (1ull << 24)) return SO_OK;   // int32 offsets up to batch 128
    w.cpw = choose_cpw(ctx, w, g.Cout, run, batch);
    const uint32_t cpw = (uint32_t)w.cpw;
    w.groups = so_ceil_div(E->m, cpw);

    // counts per (channel, chunk), then the streams
    std::vector<uint32_t> cnt((size_t)E->m * w.nch, 0);
    for (uint32_t co = 0; co < E->m; ++co)
        for (uint32_t j = 0; j < nnz[co]; ++j) ++cnt[(size_t)co * w.nch + idx[(size_t)co * E->r + j] / kHW / cc];
    std::vector<uint32_t> gbase(w.groups), quads((size_t)w.groups * w.nch * cpw, 0);
    uint64_t total_quads = 0;
    for (uint32_t gi = 0; gi < w.groups; ++gi) {
        gbase[gi] = (uint32_t)total_quads;
        for (uint32_t t = 0; t < w.nch; ++t)
            for (uint32_t c = 0; c < cpw; ++c) {
                const uint32_t co = gi * cpw + c;
                const uint32_t q = co < E->m ? (cnt[(size_t)co * w.nch + t] + 3u) / 4u : 0u;
                quads[((size_t)gi * w.nch + t) * cpw + c] = q;
                total_quads += q;
            }
        if (total_quads > 0x3fffffffull) return SO_OK;
    }
    const float neg_zero = -0.0f;
    uint32_t pad_bits;
    std::memcpy(&pad_bits, &neg_zero, 4);
    // twelve padding quads at the end: the kernels request entries one quad, or one group of 16, ahead,
    // and touch the stream's cache lines four at a time
    std::vector<int2> stream((size_t)(total_quads + 12) * 4, make_int2((int32_t)pad_bits, (int32_t)(cc * w.IH * w.IW)));
    {
        size_t pos = 0;                                            // entries written so far
        std::vector<uint32_t> next(E->m, 0);                       // next unread slot of every row
        for (uint32_t gi = 0; gi < w.groups; ++gi)
            for (uint32_t t = 0; t < w.nch; ++t)
                for (uint32_t c = 0; c < cpw; ++c) {
                    const uint32_t co = gi * cpw + c;
                    if (co >= E->m) continue;
                    const uint32_t n = cnt[(size_t)co * w.nch + t];
                    for (uint32_t e = 0; e < n; ++e) {
                        const size_t slot = (size_t)co * E->r + next[co]++;
                        const uint32_t k = idx[slot];
                        const uint32_t cin = k / kHW, kh = (k / g.kW) % g.kH, kw = k % g.kW;
                        uint32_t wb;
                        std::memcpy(&wb, &Wd[slot], 4);
                        stream[pos + e] = make_int2((int32_t)wb, (int32_t)(((cin - t * cc) * w.IH + kh * g.dil_h) * w.IW + kw * g.dil_w));
                    }
                    pos += (size_t)((n + 3u) / 4u) * 4u;
                }
    }
    void *d1 = nullptr, *d2 = nullptr, *d3 = nullptr;
    so_status s = window_configure(ctx);
    if (s != SO_OK) return s;
    s = so_malloc(ctx, stream.size() * sizeof(int2), &d1);
    if (s == SO_OK) s = so_h2d(ctx, d1, stream.data(), stream.size() * sizeof(int2));
    if (s == SO_OK) s = so_malloc(ctx, gbase.size() * sizeof(uint32_t), &d2);
    if (s == SO_OK) s = so_h2d(ctx, d2, gbase.data(), gbase.size() * sizeof(uint32_t));
    if (s == SO_OK) s = so_malloc(ctx, quads.size() * sizeof(uint32_t), &d3);
    if (s == SO_OK) s = so_h2d(ctx, d3, quads.data(), quads.size() * sizeof(uint32_t));
    if (s != SO_OK) {
        if (d1) (void)hipFree(d1);
        if (d2) (void)hipFree(d2);
        if (d3) (void)hipFree(d3);
        return s;
    }
    w.d_stream = (int2 *)d1;
    w.d_gbase = (uint32_t *)d2;
    w.d_quads = (uint32_t *)d3;
    plan->win = w;
    return SO_OK;
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
    std::vector<float> Wd(slots);
    so_status s = so_ellpack_download(ctx, E, SO_LAYOUT_ROW, Wd.data(), idx.data(), nnz.data());
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
    s = build_window(ctx, plan, idx, nnz, Wd, 32);
    if (s != SO_OK) {
        (void)hipFree(plan->d_taps);
        delete plan;
        return s;
    }
    *out = plan;
    return SO_OK;
}

static void free_window(so_conv_plan *plan)
{
    if (plan->win.d_stream) (void)hipFree(plan->win.d_stream);
    if (plan->win.d_gbase) (void)hipFree(plan->win.d_gbase);
    if (plan->win.d_quads) (void)hipFree(plan->win.d_quads);
    plan->win = so_conv_window();
}

extern "C" so_status so_conv_plan_free(so_ctx *ctx, so_conv_plan *plan)
{
    if (!plan) return SO_OK;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (plan->d_taps) (void)hipFree(plan->d_taps);
    free_window(plan);
    so_conv_rbm_release(plan);
    delete plan;
    return SO_OK;
}

extern "C" so_status so_conv_plan_tune(so_ctx *ctx, so_conv_plan *plan, uint32_t B)
{
    SO_REQUIRE(ctx && plan, "so_conv_plan_tune: null argument");
    // The layout depends on the batch only through the number of batch tiles.
    const uint32_t batch = std::max(4u, B / 4u * 4u);
    if (batch == plan->tuned_batch) return SO_OK;
    const so_ellpack *E = plan->E;
    const uint32_t lpp = window_lpp(batch) ? window_lpp(batch) : kWinLPP;
    // Rebuild only if the batch changes the batch tile the chunks are sized for or the choice of
    // channels per wave.  A plan without the layout (the geometry did not suit the batch tile tried
    // last) is tried again when the batch tile changes: a smaller tile holds more channels per chunk.
    if (plan->win.cc == 0) {
        if (lpp == plan->tried_lpp) { plan->tuned_batch = batch; return SO_OK; }
    } else {
        const double run = (double)E->total_nnz / (double)plan->g.Cout / plan->win.nch;
        if (lpp == plan->win.lpp && choose_cpw(ctx, plan->win, plan->g.Cout, run, batch) == plan->win.cpw) {
            plan->tuned_batch = batch;
            return SO_OK;
        }
    }
    const size_t slots = (size_t)E->m * E->r;
    std::vector<uint32_t> idx(slots), nnz(E->m);
    std::vector<float> Wd(slots);
    so_status s = so_ellpack_download(ctx, E, SO_LAYOUT_ROW, Wd.data(), idx.data(), nnz.data());
    if (s != SO_OK) return s;
    SO_HIP(hipStreamSynchronize(ctx->stream));      // no launch may still be reading the old arrays
    free_window(plan);
    plan->tuned_batch = batch;
    s = build_window(ctx, plan, idx, nnz, Wd, batch);
    if (s != SO_OK) return s;
    return so_conv_rbm_rebuild(ctx, plan);          // the record streams follow the window's chunks
}

extern "C" so_status so_conv_plan_window(const so_conv_plan *plan, uint32_t out[8])
{
    SO_REQUIRE(plan && out, "so_conv_plan_window: null argument");
    const so_conv_window &w = plan->win;
    const uint32_t v[8] = {w.TH, w.TW, w.IH, w.IW, w.cc, w.nch, (uint32_t)w.cpw, 0u};
    for (int i = 0; i < 8; ++i) out[i] = w.cc ? v[i] : 0u;
    return SO_OK;
}

static so_status conv2d_dispatch(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                                 const float *dBias, const float *dResid, float *dY, int act)
{
    SO_REQUIRE(ctx && plan, "so_conv2d: null argument");
    SO_REQUIRE(act >= SO_ACT_NONE && act <= SO_ACT_TANH, "so_conv2d: unknown activation %d", act);
    const so_conv_geom &g = plan->g;
    const uint64_t ncols = (uint64_t)g.H_out * g.W_out * B;
    if (g.Cout == 0 || ncols == 0) return SO_OK;
    SO_REQUIRE(dX && dY, "so_conv2d: null tensor");
    SO_REQUIRE((ncols + 63) / 64 < (1ull << 31), "so_conv2d: output plane too large");
    // Batch entries per lane: as many as divide B and keep 16/8-byte alignment.
    const uintptr_t align = (uintptr_t)dX | (uintptr_t)dY | (uintptr_t)dResid;
    int maxvec = 4;
    if (ctx->tune.conv_vec > 0) maxvec = ctx->tune.conv_vec;
    // The LDS-windowed kernel when the plan carries its layout and the batch splits into tiles of
    // 16, 8 or 4 (SPARSEOPS_CONV_WINDOW=1 forces it whenever possible, =0 forbids it: tuning and tests).
    const uint32_t lpp = window_lpp(B);
    if (plan->win.cc != 0 && lpp != 0 && (align & 15) == 0 && (uint64_t)plan->win.cc * g.H_in * g.W_in * B < (1ull << 31)) {
        // a plan that carries the row-block-merged streams runs that kernel (SPARSEOPS_CONV_RBM=0 forbids it).  It is an
        // LDS-windowed kernel itself: SPARSEOPS_CONV_WINDOW=0 forbids it too, unless SPARSEOPS_CONV_RBM=1 asks for it.
        if (plan->rbm.d_sets && ctx->tune.conv_rbm != 0 && (ctx->tune.conv_window != 0 || ctx->tune.conv_rbm == 1)) {
            bool done = false;
            const so_status s = so_conv_rbm_launch(ctx, plan, dX, B, dBias, dResid, dY, act, ctx->tune.conv_rbm == 1, &done);
            if (s != SO_OK) return s;
            if (done) {
                SO_LAUNCH_CHECK();
                return SO_OK;
            }
        }
        const bool forced = ctx->tune.conv_window == 1;
        if (ctx->tune.conv_window != 0) {
            bool done = false;
            const so_status s = lpp == 4 ? window_launch<4>(ctx, plan, dX, B, dBias, dResid, dY, act, forced, &done)
                              : lpp == 2 ? window_launch<2>(ctx, plan, dX, B, dBias, dResid, dY, act, forced, &done)
                                         : window_launch<1>(ctx, plan, dX, B, dBias, dResid, dY, act, forced, &done);
            if (s != SO_OK) return s;
            if (done) {
                SO_LAUNCH_CHECK();
                return SO_OK;
            }
        }
    }
    if (maxvec >= 4 && B % 4 == 0 && (align & 15) == 0) conv_launch<4>(ctx, plan, dX, B, ncols, dBias, dResid, dY, act);
    else if (maxvec >= 2 && B % 2 == 0 && (align & 7) == 0) conv_launch<2>(ctx, plan, dX, B, ncols, dBias, dResid, dY, act);
    else conv_launch<1>(ctx, plan, dX, B, ncols, dBias, dResid, dY, act);
    SO_LAUNCH_CHECK();
    return SO_OK;
}

extern "C" so_status so_conv2d(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                               const float *dBias, float *dY, int act)
{
    return conv2d_dispatch(ctx, plan, dX, B, dBias, nullptr, dY, act);
}

extern "C" so_status so_conv2d_add(so_ctx *ctx, const so_conv_plan *plan, const float *dX, uint32_t B,
                                   const float *dBias, const float *dResidual, float *dY, int act)
{
    SO_REQUIRE(dResidual, "so_conv2d_add: null residual");
    SO_REQUIRE(dResidual != dY, "so_conv2d_add: the residual must not alias the output");
    return conv2d_dispatch(ctx, plan, dX, B, dBias, dResidual, dY, act);
}
