// Micro-benchmark behind the operand-delivery ceilings quoted for the LDS-fed kernels: how many
// bytes per clock a compute unit can take out of LDS with ds_read_b128 / b64 / b32 (conflict-free,
// 16 waves per CU, nothing else going on), and how many fp32 multiply-adds per clock it retires
// with plain v_fma_f32 and with the DPP form the kernels use, alone and combined in the kernels' own
// step loop.  Clocks are the shader clock (s_memtime) read inside the kernel by every
// wave: a wave's cycles run from its first to its last instruction, a CU's figure uses the longest.
//
//   make -C sparse-ops_amd bench/lds_probe && sparse-ops_amd/bench/lds_probe
#include <hip/hip_runtime.h>

#include "dpp_steps.h"
#include "conv_internal.h"

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("%s: %s\n", #x, hipGetErrorString(e_)); std::exit(1); } } while (0)

constexpr int kThreads = 1024;   // 16 waves: one workgroup per CU
constexpr int kIters = 2048;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// One step with the (weight, offset) pair of lane N of each 16-lane row: variants of how the pair
// reaches the lanes.  V2: two 32-bit DPP moves/adds + plain multiply-adds.  V3: one 64-bit DPP move.
template <int N>
__device__ __forceinline__ void step_v2_addr(uint32_t base, uint32_t eo, uint32_t &addr)
{
    asm volatile("v_add_u32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf" : "=v"(addr) : "v"(eo), "v"(base), "n"(N));
}
template <int N>
__device__ __forceinline__ float step_v2_w(float ew)
{
    float w;
    asm volatile("v_mov_b32_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(w) : "v"(ew), "n"(N));
    return w;
}
template <int N>
__device__ __forceinline__ u32x2 step_v3_pair(u32x2 e)
{
    u32x2 r;
    asm volatile("v_mov_b64_dpp %0, %1 row_newbcast:%2 row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(e), "n"(N));
    return r;
}
__device__ __forceinline__ void fma4(float (&a)[4], float w, const f32x4 &x)
{
    a[0] = __builtin_fmaf(w, x.x, a[0]); a[1] = __builtin_fmaf(w, x.y, a[1]);
    a[2] = __builtin_fmaf(w, x.z, a[2]); a[3] = __builtin_fmaf(w, x.w, a[3]);
}
template <int N0>
__device__ __forceinline__ void steps8_v2(const char *lds, uint32_t base, float ew, uint32_t eo, float (&a)[4])
{
    f32x4 x[8];
    uint32_t ad[8];
    step_v2_addr<N0 + 0>(base, eo, ad[0]); step_v2_addr<N0 + 1>(base, eo, ad[1]); step_v2_addr<N0 + 2>(base, eo, ad[2]);
    step_v2_addr<N0 + 3>(base, eo, ad[3]); step_v2_addr<N0 + 4>(base, eo, ad[4]); step_v2_addr<N0 + 5>(base, eo, ad[5]);
    step_v2_addr<N0 + 6>(base, eo, ad[6]); step_v2_addr<N0 + 7>(base, eo, ad[7]);
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = *reinterpret_cast<const f32x4 *>(lds + ad[u]);
    fma4(a, step_v2_w<N0 + 0>(ew), x[0]); fma4(a, step_v2_w<N0 + 1>(ew), x[1]); fma4(a, step_v2_w<N0 + 2>(ew), x[2]);
    fma4(a, step_v2_w<N0 + 3>(ew), x[3]); fma4(a, step_v2_w<N0 + 4>(ew), x[4]); fma4(a, step_v2_w<N0 + 5>(ew), x[5]);
    fma4(a, step_v2_w<N0 + 6>(ew), x[6]); fma4(a, step_v2_w<N0 + 7>(ew), x[7]);
}
template <int N0>
__device__ __forceinline__ void steps8_v3(const char *lds, uint32_t base, u32x2 e, float (&a)[4])
{
    f32x4 x[8];
    u32x2 p[8];
    p[0] = step_v3_pair<N0 + 0>(e); p[1] = step_v3_pair<N0 + 1>(e); p[2] = step_v3_pair<N0 + 2>(e); p[3] = step_v3_pair<N0 + 3>(e);
    p[4] = step_v3_pair<N0 + 4>(e); p[5] = step_v3_pair<N0 + 5>(e); p[6] = step_v3_pair<N0 + 6>(e); p[7] = step_v3_pair<N0 + 7>(e);
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = *reinterpret_cast<const f32x4 *>(lds + base + p[u].y);
#pragma unroll
    for (int u = 0; u < 8; ++u) fma4(a, __builtin_bit_cast(float, p[u].x), x[u]);
}

// MODE 0/1/2: 8 ds_read_b128 / b64 / b32 per iteration (inline asm, so that none is merged or hoisted),
//             each lane its own 16 / 8 / 4 bytes (consecutive lanes, consecutive addresses: no bank
//             conflict), results never used.
// MODE 18/20/21: 8 ds_write_b128 / b64 / b32 per iteration.
// MODE 19:    8 ds_read_b128 per iteration, every lane at an address of its own (bank-conflict patterns).
// MODE 3:     32 independent v_fma_f32 per iteration, no memory access.
// MODE 23:    32 v_fmac_f32 per iteration on one accumulator (a dependent chain).
// MODE 4:     32 v_fmac_f32_dpp row_newbcast per iteration (the multiply-add of the LDS-fed kernels' steps).
// MODE 5:     the step loop of the tiled matmul and the windowed convolution itself (csrc/dpp_steps.h):
//             16 steps per iteration, each one ds_read_b128 + one address add + four multiply-adds.
// MODE 6:     the same steps with the weight moved by a 32-bit DPP move and plain multiply-adds.
// MODE 7:     the same steps with (weight, offset) moved together by one 64-bit DPP move.
// MODE 8:     steps whose weight and offset are wave-uniform scalars (no loads: the ceiling of that form).
// MODE 9:     wave-uniform entries read from LDS (every lane the same 16 bytes = two entries) into vector registers.
// MODE 11:    MODE 9 with a different address for each of the wave's four 16-lane rows.
// MODE 10:    wave-uniform entries read from memory with a vector load of one address (16 bytes = two entries).
template <int MODE>
__global__ __launch_bounds__(kThreads) void probe(float *out, unsigned long long *cycles, const uint32_t *offs, const float *gents)
{
    extern __shared__ float4 lds[];
    const uint32_t tid = threadIdx.x;
    for (uint32_t i = tid; i < 8192; i += blockDim.x) lds[i] = make_float4(1.f, 2.f, 3.f, 4.f);
    // behind the 64 KB of "X": 64 wave-uniform entries {weight, byte offset, weight, byte offset}
    for (uint32_t i = tid; i < 320; i += blockDim.x)
        lds[4096 + i] = make_float4(1.5f, __builtin_bit_cast(float, (i * 37u % 60u) * 1024u), 0.5f, __builtin_bit_cast(float, (i * 11u % 60u) * 1024u));
    __syncthreads();
    float acc = 0.f;
    float r[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) r[j] = (float)(tid + j);
    const uint32_t addr = (tid & 63u) * ((MODE == 0 || MODE == 18) ? 16u : (MODE == 1 || MODE == 20) ? 8u : 4u) + (tid >> 6) * 4096u;
    float a4[4] = {0.f, 0.f, 0.f, 0.f};
    const uint32_t eo = offs[tid & 63u];                  // per-lane step offsets (multiples of 256 below 16 KB)
    const float ew = 1.0f + (float)(tid & 15u);
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < kIters; ++it) {
        if constexpr (MODE == 0) {
            f32x4 x0, x1, x2, x3, x4, x5, x6, x7;
            asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:1024\n\tds_read_b128 %2, %8 offset:2048\n\t"
                         "ds_read_b128 %3, %8 offset:3072\n\tds_read_b128 %4, %8\n\tds_read_b128 %5, %8 offset:1024\n\t"
                         "ds_read_b128 %6, %8 offset:2048\n\tds_read_b128 %7, %8 offset:3072\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(x0), "=&v"(x1), "=&v"(x2), "=&v"(x3), "=&v"(x4), "=&v"(x5), "=&v"(x6), "=&v"(x7) : "v"(addr));
        } else if constexpr (MODE == 1) {
            f32x2 x0, x1, x2, x3, x4, x5, x6, x7;
            asm volatile("ds_read_b64 %0, %8\n\tds_read_b64 %1, %8 offset:512\n\tds_read_b64 %2, %8 offset:1024\n\t"
                         "ds_read_b64 %3, %8 offset:1536\n\tds_read_b64 %4, %8\n\tds_read_b64 %5, %8 offset:512\n\t"
                         "ds_read_b64 %6, %8 offset:1024\n\tds_read_b64 %7, %8 offset:1536\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(x0), "=&v"(x1), "=&v"(x2), "=&v"(x3), "=&v"(x4), "=&v"(x5), "=&v"(x6), "=&v"(x7) : "v"(addr));
        } else if constexpr (MODE == 2) {
            float x0, x1, x2, x3, x4, x5, x6, x7;
            asm volatile("ds_read_b32 %0, %8\n\tds_read_b32 %1, %8 offset:256\n\tds_read_b32 %2, %8 offset:512\n\t"
                         "ds_read_b32 %3, %8 offset:768\n\tds_read_b32 %4, %8\n\tds_read_b32 %5, %8 offset:256\n\t"
                         "ds_read_b32 %6, %8 offset:512\n\tds_read_b32 %7, %8 offset:768\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(x0), "=&v"(x1), "=&v"(x2), "=&v"(x3), "=&v"(x4), "=&v"(x5), "=&v"(x6), "=&v"(x7) : "v"(addr));
        } else if constexpr (MODE == 19) {
            // ds_read_b128 with this lane's address taken from a table: which lane groups share a turn of the banks
            f32x4 x0, x1, x2, x3, x4, x5, x6, x7;
            asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:16384\n\tds_read_b128 %2, %8 offset:32768\n\t"
                         "ds_read_b128 %3, %8 offset:49152\n\tds_read_b128 %4, %8\n\tds_read_b128 %5, %8 offset:16384\n\t"
                         "ds_read_b128 %6, %8 offset:32768\n\tds_read_b128 %7, %8 offset:49152\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(x0), "=&v"(x1), "=&v"(x2), "=&v"(x3), "=&v"(x4), "=&v"(x5), "=&v"(x6), "=&v"(x7) : "v"(eo));
        } else if constexpr (MODE == 18) {
            f32x4 v = {1.f, 2.f, 3.f, (float)it};
            asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %1 offset:1024\n\tds_write_b128 %0, %1 offset:2048\n\t"
                         "ds_write_b128 %0, %1 offset:3072\n\tds_write_b128 %0, %1\n\tds_write_b128 %0, %1 offset:1024\n\t"
                         "ds_write_b128 %0, %1 offset:2048\n\tds_write_b128 %0, %1 offset:3072\n\ts_waitcnt lgkmcnt(0)"
                         : : "v"(addr), "v"(v) : "memory");
        } else if constexpr (MODE == 22) {
            // the same with every write of an iteration at another address (8 KB per wave)
            f32x4 v = {1.f, 2.f, 3.f, (float)it};
            const uint32_t a8 = (tid & 63u) * 16u + (tid >> 6) * 8192u;
            asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %1 offset:1024\n\tds_write_b128 %0, %1 offset:2048\n\t"
                         "ds_write_b128 %0, %1 offset:3072\n\tds_write_b128 %0, %1 offset:4096\n\tds_write_b128 %0, %1 offset:5120\n\t"
                         "ds_write_b128 %0, %1 offset:6144\n\tds_write_b128 %0, %1 offset:7168\n\ts_waitcnt lgkmcnt(0)"
                         : : "v"(a8), "v"(v) : "memory");
        } else if constexpr (MODE == 20) {
            f32x2 v = {1.f, (float)it};
            asm volatile("ds_write_b64 %0, %1\n\tds_write_b64 %0, %1 offset:512\n\tds_write_b64 %0, %1 offset:1024\n\t"
                         "ds_write_b64 %0, %1 offset:1536\n\tds_write_b64 %0, %1\n\tds_write_b64 %0, %1 offset:512\n\t"
                         "ds_write_b64 %0, %1 offset:1024\n\tds_write_b64 %0, %1 offset:1536\n\ts_waitcnt lgkmcnt(0)"
                         : : "v"(addr), "v"(v) : "memory");
        } else if constexpr (MODE == 21) {
            float v = (float)it;
            asm volatile("ds_write_b32 %0, %1\n\tds_write_b32 %0, %1 offset:256\n\tds_write_b32 %0, %1 offset:512\n\t"
                         "ds_write_b32 %0, %1 offset:768\n\tds_write_b32 %0, %1\n\tds_write_b32 %0, %1 offset:256\n\t"
                         "ds_write_b32 %0, %1 offset:512\n\tds_write_b32 %0, %1 offset:768\n\ts_waitcnt lgkmcnt(0)"
                         : : "v"(addr), "v"(v) : "memory");
        } else if constexpr (MODE == 3) {
            const float w = (float)it;
#pragma unroll
            for (int j = 0; j < 32; ++j) r[j] = __builtin_fmaf(w, r[j], 1.0f);
        } else if constexpr (MODE == 12 || MODE == 13) {
            // acc += w * x with all three in vector registers (12) or the weight in a scalar register (13)
            const float wv = MODE == 12 ? ew + (float)it : __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, ew + (float)it)));
#pragma unroll
            for (int j = 0; j < 16; ++j) r[j] = __builtin_fmaf(wv, r[16 + j], r[j]);
#pragma unroll
            for (int j = 0; j < 16; ++j) r[j] = __builtin_fmaf(wv, r[31 - j], r[j]);
        } else if constexpr (MODE == 23) {
            // one chain: every multiply-add waits for the one before it
            const float wv = 1.0f + 1e-7f * (float)it;
#pragma unroll
            for (int j = 0; j < 32; ++j) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(r[0]) : "v"(wv), "v"(r[1 + (j & 15)]));
        } else if constexpr (MODE == 4) {
#pragma unroll
            for (int j = 0; j < 32; ++j)
                asm volatile("v_fmac_f32_dpp %0, %1, %2 row_newbcast:3 row_mask:0xf bank_mask:0xf" : "+v"(r[j]) : "v"(ew), "v"(acc));
        } else if constexpr (MODE == 5) {
            const uint32_t o = eo + (uint32_t)(it & 3) * 64u;       // the reads change from iteration to iteration
            so_dpp::tiled_chunk((const char *)lds + (tid & 15u) * 16u, ew, o, 16u, a4);
        } else if constexpr (MODE == 6) {
            uint32_t o = eo + (uint32_t)(it & 3) * 64u;
            asm volatile("s_nop 4" : "+v"(o));          // a DPP source must not have been written in the last two cycles
            steps8_v2<0>((const char *)lds, (tid & 15u) * 16u, ew, o, a4);
            steps8_v2<8>((const char *)lds, (tid & 15u) * 16u, ew, o, a4);
        } else if constexpr (MODE == 7) {
            u32x2 e;
            e.x = __builtin_bit_cast(uint32_t, ew);
            e.y = eo + (uint32_t)(it & 3) * 64u;
            asm volatile("s_nop 4" : "+v"(e));
            steps8_v3<0>((const char *)lds, (tid & 15u) * 16u, e, a4);
            steps8_v3<8>((const char *)lds, (tid & 15u) * 16u, e, a4);
        } else if constexpr (MODE == 8) {
            const uint32_t so = __builtin_amdgcn_readfirstlane(eo) + (uint32_t)(it & 3) * 64u;
            const float sw = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, ew)));
            f32x4 x[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) x[u] = *reinterpret_cast<const f32x4 *>((const char *)lds + (tid & 63u) * 16u + so + u * 1024u);
#pragma unroll
            for (int u = 0; u < 16; ++u) fma4(a4, sw + (float)u, x[u]);
        } else if constexpr (MODE == 9 || MODE == 11 || MODE == 17) {
            // 8 broadcast reads = 16 entries {w, off, w, off}, then the 16 steps (MODE 11: every 16-lane row its own entries)
            const char *ents = (const char *)lds + 65536 + (uint32_t)(it & 7) * 128u + (MODE != 9 ? ((tid >> 4) & 3u) * 1040u : 0u);
            const uint32_t xl = MODE == 17 ? (tid & 15u) * 16u : (tid & 63u) * 16u;   // 17: the four rows read the same 256-byte column range of different X rows
            float4 e[8], x[16];                  // HIP's float4: element access on clang's vector type was merged by the compiler
#pragma unroll
            for (int u = 0; u < 8; ++u) e[u] = *reinterpret_cast<const float4 *>(ents + u * 16);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                x[2 * u] = *reinterpret_cast<const float4 *>((const char *)lds + xl + __float_as_uint(e[u].y));
                x[2 * u + 1] = *reinterpret_cast<const float4 *>((const char *)lds + xl + __float_as_uint(e[u].w));
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                a4[0] = __builtin_fmaf(e[u].x, x[2 * u].x, a4[0]); a4[1] = __builtin_fmaf(e[u].x, x[2 * u].y, a4[1]);
                a4[2] = __builtin_fmaf(e[u].x, x[2 * u].z, a4[2]); a4[3] = __builtin_fmaf(e[u].x, x[2 * u].w, a4[3]);
                a4[0] = __builtin_fmaf(e[u].z, x[2 * u + 1].x, a4[0]); a4[1] = __builtin_fmaf(e[u].z, x[2 * u + 1].y, a4[1]);
                a4[2] = __builtin_fmaf(e[u].z, x[2 * u + 1].z, a4[2]); a4[3] = __builtin_fmaf(e[u].z, x[2 * u + 1].w, a4[3]);
            }
        } else {
            const float4 *ents = reinterpret_cast<const float4 *>(gents) + (size_t)(blockIdx.x & 31u) * 64 + (uint32_t)(it & 7) * 8u;
            float4 e[8], x[16];
#pragma unroll
            for (int u = 0; u < 8; ++u) e[u] = ents[u];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                x[2 * u] = *reinterpret_cast<const float4 *>((const char *)lds + (tid & 63u) * 16u + __float_as_uint(e[u].y));
                x[2 * u + 1] = *reinterpret_cast<const float4 *>((const char *)lds + (tid & 63u) * 16u + __float_as_uint(e[u].w));
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                a4[0] = __builtin_fmaf(e[u].x, x[2 * u].x, a4[0]); a4[1] = __builtin_fmaf(e[u].x, x[2 * u].y, a4[1]);
                a4[2] = __builtin_fmaf(e[u].x, x[2 * u].z, a4[2]); a4[3] = __builtin_fmaf(e[u].x, x[2 * u].w, a4[3]);
                a4[0] = __builtin_fmaf(e[u].z, x[2 * u + 1].x, a4[0]); a4[1] = __builtin_fmaf(e[u].z, x[2 * u + 1].y, a4[1]);
                a4[2] = __builtin_fmaf(e[u].z, x[2 * u + 1].z, a4[2]); a4[3] = __builtin_fmaf(e[u].z, x[2 * u + 1].w, a4[3]);
            }
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
#pragma unroll
    for (int j = 0; j < 32; ++j) acc += r[j];
    out[(size_t)blockIdx.x * kThreads + tid] = acc + a4[0] + a4[1] + a4[2] + a4[3];
    if ((tid & 63u) == 0) {
        cycles[((size_t)blockIdx.x * 16 + (tid >> 6)) * 2] = t0;
        cycles[((size_t)blockIdx.x * 16 + (tid >> 6)) * 2 + 1] = t1;
    }
}

template <int MODE>
void run(const char *what, int cus, int waves, double per_wave_iter, const char *unit, float *dOut, unsigned long long *dCyc,
         const uint32_t *dOffs, const float *dEnts)
{
    CK(hipFuncSetAttribute((const void *)probe<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    std::vector<unsigned long long> cyc((size_t)cus * 32);
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int rep = 0; rep < 3; ++rep) probe<MODE><<<cus, waves * 64, 131072>>>(dOut, dCyc, dOffs, dEnts);   // clocks up
    CK(hipEventRecord(e0));
    probe<MODE><<<cus, waves * 64, 131072>>>(dOut, dCyc, dOffs, dEnts);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms = 0;
    CK(hipEventElapsedTime(&ms, e0, e1));
    CK(hipMemcpy(cyc.data(), dCyc, cyc.size() * 8, hipMemcpyDeviceToHost));
    // per CU: from the earliest start to the latest end of its 16 waves
    std::vector<double> per_cu;
    for (int b = 0; b < cus; ++b) {
        unsigned long long lo = ~0ull, hi = 0;
        for (int w = 0; w < waves; ++w) { lo = std::min(lo, cyc[(b * 16 + w) * 2]); hi = std::max(hi, cyc[(b * 16 + w) * 2 + 1]); }
        per_cu.push_back(double(waves) * kIters * per_wave_iter / double(hi - lo));
    }
    std::sort(per_cu.begin(), per_cu.end());
    std::printf("%-58s %2d waves/CU %8.1f %s per clock and CU (median of %d CUs; min %.1f, max %.1f); launch %.1f us\n", what, waves,
                per_cu[per_cu.size() / 2], unit, cus, per_cu.front(), per_cu.back(), ms * 1e3);
}

int main()
{
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    std::printf("%s, %d CUs, clock rate %d kHz\n", prop.gcnArchName, cus, prop.clockRate);
    float *dOut;
    unsigned long long *dCyc;
    CK(hipMalloc(&dOut, (size_t)cus * kThreads * 4));
    CK(hipMalloc(&dCyc, (size_t)cus * 32 * 8));
    std::vector<uint32_t> offs(64);
    for (int i = 0; i < 64; ++i) offs[i] = (uint32_t)((i * 37) % 60) * 256u;      // X rows of a 64-column tile, any order
    uint32_t *dOffs;
    CK(hipMalloc(&dOffs, 256));
    CK(hipMemcpy(dOffs, offs.data(), 256, hipMemcpyHostToDevice));
    std::vector<float> ents(32 * 64 * 4);
    for (size_t i = 0; i < ents.size() / 4; ++i) {
        const uint32_t o0 = (uint32_t)(i * 37 % 60) * 1024u, o1 = (uint32_t)(i * 11 % 60) * 1024u;
        ents[4 * i] = 1.5f; std::memcpy(&ents[4 * i + 1], &o0, 4); ents[4 * i + 2] = 0.5f; std::memcpy(&ents[4 * i + 3], &o1, 4);
    }
    float *dEnts;
    CK(hipMalloc(&dEnts, ents.size() * 4));
    CK(hipMemcpy(dEnts, ents.data(), ents.size() * 4, hipMemcpyHostToDevice));
    // ds_read_b128 address patterns (byte address of each lane inside a 16 KB region)
    {
        struct { const char *what; uint32_t (*addr)(uint32_t); } pats[] = {
            {"64 lanes x 16 B contiguous", [](uint32_t l) { return l * 16u; }},
            {"4 groups of 16 lanes, each 256 B contiguous, all on the same banks", [](uint32_t l) { return (l % 16u) * 16u + (l / 16u) * 4096u; }},
            {"8 groups of 8 lanes, each 128 B contiguous, all on banks 0-31", [](uint32_t l) { return (l % 8u) * 16u + (l / 8u) * 2048u; }},
            {"8 groups of 8 lanes, odd groups on banks 32-63", [](uint32_t l) { return (l % 8u) * 16u + ((l / 8u) & 1u) * 128u + (l / 8u) * 2048u; }},
            {"16 groups of 4 lanes (64 B), all on banks 0-15", [](uint32_t l) { return (l % 4u) * 16u + (l / 4u) * 1024u; }},
            {"16 groups of 4 lanes, group g on bank group g mod 4", [](uint32_t l) { return (l % 4u) * 16u + ((l / 4u) & 3u) * 64u + (l / 4u) * 1024u; }},
            {"16 groups of 4 lanes, bank groups 0,0,1,1,2,2,3,3 repeated", [](uint32_t l) { return (l % 4u) * 16u + (((l / 4u) >> 1) & 3u) * 64u + (l / 4u) * 1024u; }},
            {"16 groups of 4 lanes, bank groups 0,1,2,3,3,2,1,0 ...", [](uint32_t l) { const uint32_t g = l / 4u; return (l % 4u) * 16u + (((g & 4u) ? 3u - (g & 3u) : (g & 3u))) * 64u + g * 1024u; }},
            {"tile 4x7 pixels in a 9-pixel-wide window, row-major slots", [](uint32_t l) { const uint32_t p = l / 4u; return (l % 4u) * 16u + ((p / 7u) * 9u + p % 7u) * 64u; }},
        };
        for (auto &pt : pats) {
            for (int i = 0; i < 64; ++i) offs[i] = pt.addr((uint32_t)i);
            CK(hipMemcpy(dOffs, offs.data(), 256, hipMemcpyHostToDevice));
            run<19>(pt.what, cus, 16, 8.0 * 64 * 16, "bytes (ds_read_b128)", dOut, dCyc, dOffs, dEnts);
        }
        // the windowed convolution's reads: 4 lanes per output pixel (16 batch entries), 16 pixels per wave; tiles of
        // the ResNet-18-shaped layers, pixel slots in row-major order and in the order window_pixel_order deals them
        struct { const char *what; uint32_t TH, TW, IW, sth, stw; } tiles[] = {
            {"tile 4x8, window row 10 pixels (56x56 3x3 layers)", 4, 8, 10, 1, 1},
            {"tile 4x7, window row 9 (28x28 3x3 layers)", 4, 7, 9, 1, 1},
            {"tile 2x7, window row 9 (14x14 and 7x7 3x3 layers)", 2, 7, 9, 1, 1},
            {"tile 4x7, stride 2, window row 15 (3x3 stride-2 layers)", 4, 7, 15, 2, 2},
            {"tile 4x8, stride 2, window row 21 (7x7 stride-2 stem)", 4, 8, 21, 2, 2},
        };
        for (auto &t : tiles)
            for (int permuted = 0; permuted < 2; ++permuted)
                for (uint32_t wave = 0; wave * 16u < t.TH * t.TW; ++wave) {
                    WinArgs a{};
                    a.TH = t.TH; a.TW = t.TW; a.IW = t.IW; a.sth = t.sth; a.stw = t.stw;
                    window_pixel_order(a, 4);
                    for (uint32_t l = 0; l < 64; ++l) {
                        const uint32_t slot = wave * 16u + l / 4u;
                        uint32_t px = slot < t.TH * t.TW ? slot : 0u;
                        if (permuted) px = (a.order[slot >> 2] >> ((slot & 3u) * 8u)) & 0xffu;
                        offs[l] = (l % 4u) * 16u + ((px / t.TW) * t.sth * t.IW + (px % t.TW) * t.stw) * 64u;
                    }
                    CK(hipMemcpy(dOffs, offs.data(), 256, hipMemcpyHostToDevice));
                    char what[160];
                    std::snprintf(what, sizeof what, "%s, wave %u, %s", t.what, wave, permuted ? "dealt slots" : "row-major slots");
                    run<19>(what, cus, 16, 8.0 * 64 * 16, "bytes (ds_read_b128)", dOut, dCyc, dOffs, dEnts);
                }
        for (int i = 0; i < 64; ++i) offs[i] = (uint32_t)((i * 37) % 60) * 256u;
        CK(hipMemcpy(dOffs, offs.data(), 256, hipMemcpyHostToDevice));
    }
    // one wave per SIMD, one chain: 256 multiply-adds per CU in flight, so clocks from one multiply-add to the next that
    // uses its result = 256 / the rate printed
    run<23>("v_fmac_f32, one dependent chain per lane", cus, 4, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
    run<23>("v_fmac_f32, one dependent chain per lane", cus, 8, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
    for (int waves : {16, 8}) {
        run<0>("ds_read_b128, conflict-free", cus, waves, 8.0 * 64 * 16, "bytes", dOut, dCyc, dOffs, dEnts);
        run<18>("ds_write_b128, conflict-free", cus, waves, 8.0 * 64 * 16, "bytes", dOut, dCyc, dOffs, dEnts);
        run<22>("ds_write_b128, conflict-free, 8 addresses per lane", cus, waves, 8.0 * 64 * 16, "bytes", dOut, dCyc, dOffs, dEnts);
        run<20>("ds_write_b64, conflict-free", cus, waves, 8.0 * 64 * 8, "bytes", dOut, dCyc, dOffs, dEnts);
        run<21>("ds_write_b32, conflict-free", cus, waves, 8.0 * 64 * 4, "bytes", dOut, dCyc, dOffs, dEnts);
        run<1>("ds_read_b64, conflict-free", cus, waves, 8.0 * 64 * 8, "bytes", dOut, dCyc, dOffs, dEnts);
        run<2>("ds_read_b32, conflict-free", cus, waves, 8.0 * 64 * 4, "bytes", dOut, dCyc, dOffs, dEnts);
        run<3>("v_fma_f32, 32 independent chains", cus, waves, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<12>("v_fmac_f32 acc += w * x, three vector registers", cus, waves, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<13>("v_fmac_f32 acc += w * x, w in a scalar register", cus, waves, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<4>("v_fmac_f32_dpp row_newbcast, 32 independent chains", cus, waves, 32.0 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<5>("step loop: ds_read_b128 + address add + 4 v_fmac_f32_dpp", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<6>("step loop: 32-bit DPP move of the weight, plain multiply-adds", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<7>("step loop: one 64-bit DPP move of (weight, offset)", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<8>("step loop: wave-uniform weight and offset in scalar registers", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<9>("step loop: wave-uniform entries read from LDS (16 B, 2 entries)", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<11>("step loop: entries read from LDS, one address per 16-lane row", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<17>("step loop: entries from LDS per row, rows read one 256-byte column range", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
        run<10>("step loop: wave-uniform entries from a one-address vector load", cus, waves, 16.0 * 4 * 64, "multiply-adds", dOut, dCyc, dOffs, dEnts);
    }
    return 0;
}
