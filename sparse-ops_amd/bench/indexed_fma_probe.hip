// Micro-benchmark behind the row-block-merged matmul's step loop (csrc/matmul_rbm.hip): the rate of
// fp32 multiply-adds whose accumulator register is chosen at run time (VGPR index mode: one M0 write
// per multiply-add, the weight a scalar operand), against the plain v_fmac with a scalar weight, at
// 16, 12 and 8 waves per compute unit, and with the records streamed through scalar loads and the
// dense operand through buffer loads as the kernel does.  Not part of the product build:
//     make -C sparse-ops_amd probe && sparse-ops_amd/bench/indexed_fma_probe
// Clock counts are shader clocks read inside the kernel (median wave); the clock the chip holds under
// the load is printed beside them (shader clocks per tick of the constant 100 MHz counter).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <vector>
#include <algorithm>
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::printf("%s: %s\n", #x, hipGetErrorString(e_)); std::exit(1); } } while (0)

typedef float f32x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define SCLOB "s36", "s37", "s38", "s39", "s40", "s41", "s42", "s43", "s44", "s45", "s46", "s47", "s48", "s49", "s50", "s51", \
              "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67"

// a set = 16 dwords: w0..w9, h01, h23, h45, h67, h89 (M0 values, two 16-bit halves each), xoff
// 10 pairs from window at S (weights S..S+9, halves S+10..S+14), x registers XA (pairs 0-4), XB (pairs 5-9)
#define PAIR_LO(W, H, X) "s_mov_b32 m0, s" #H "\n\t" "v_fmac_f32 v48, s" #W ", v" #X "\n\t"
#define PAIR_HI(W, H, X) "s_lshr_b32 m0, s" #H ", 16\n\t" "v_fmac_f32 v48, s" #W ", v" #X "\n\t"
#define SET10(W0, W1, W2, W3, W4, W5, W6, W7, W8, W9, H0, H1, H2, H3, H4, XA, XB) \
    PAIR_LO(W0, H0, XA) PAIR_HI(W1, H0, XA) PAIR_LO(W2, H1, XA) PAIR_HI(W3, H1, XA) PAIR_LO(W4, H2, XA) \
    PAIR_HI(W5, H2, XB) PAIR_LO(W6, H3, XB) PAIR_HI(W7, H3, XB) PAIR_LO(W8, H4, XB) PAIR_HI(W9, H4, XB)
#define SET_A(XA, XB) SET10(36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47, 48, 49, 50, XA, XB)
#define SET_B(XA, XB) SET10(52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63, 64, 65, 66, XA, XB)

template <int MODE>
__global__ void probe(float *out, unsigned long long *cycles, const int4 *stream, const float *X, uint32_t iters, uint32_t xbytes)
{
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nw = blockDim.x >> 6;
    f32x32 a0, a1;
#pragma unroll
    for (int i = 0; i < 32; ++i) { a0[i] = (float)(tid + i); a1[i] = (float)(tid * 2 + i); }
    float x0 = (float)lane * 0.001f;
    const int4 *sp = stream + (size_t)(blockIdx.x * nw + wave) * 4096;   // 64 KB per wave
    uint32_t cnt = iters;
    const uint32_t voff = lane * 4u;
    u32x4 rs;
    {
        const uint64_t b = (uint64_t)X;
        rs[0] = (uint32_t)b; rs[1] = (uint32_t)(b >> 32) & 0xffffu; rs[2] = xbytes; rs[3] = 0x00020000u;
    }
    rs[0] = __builtin_amdgcn_readfirstlane(rs[0]); rs[1] = __builtin_amdgcn_readfirstlane(rs[1]);
    rs[2] = __builtin_amdgcn_readfirstlane(rs[2]); rs[3] = __builtin_amdgcn_readfirstlane(rs[3]);
    __syncthreads();
    const unsigned long long r0 = wall_clock64();
    const unsigned long long t0 = __builtin_readcyclecounter();
    if constexpr (MODE == 1) {          // 20 static v_fmac per iteration
        asm volatile(
            "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
            "s_waitcnt lgkmcnt(0)\n"
            "L1_%=:\n\t"
            "v_fmac_f32 v48, s36, %[x0]\n\t" "v_fmac_f32 v52, s37, %[x0]\n\t" "v_fmac_f32 v56, s38, %[x0]\n\t" "v_fmac_f32 v60, s39, %[x0]\n\t"
            "v_fmac_f32 v64, s40, %[x0]\n\t" "v_fmac_f32 v68, s41, %[x0]\n\t" "v_fmac_f32 v72, s42, %[x0]\n\t" "v_fmac_f32 v76, s43, %[x0]\n\t"
            "v_fmac_f32 v80, s44, %[x0]\n\t" "v_fmac_f32 v84, s45, %[x0]\n\t" "v_fmac_f32 v88, s36, %[x0]\n\t" "v_fmac_f32 v92, s37, %[x0]\n\t"
            "v_fmac_f32 v96, s38, %[x0]\n\t" "v_fmac_f32 v100, s39, %[x0]\n\t" "v_fmac_f32 v104, s40, %[x0]\n\t" "v_fmac_f32 v108, s41, %[x0]\n\t"
            "v_fmac_f32 v49, s42, %[x0]\n\t" "v_fmac_f32 v53, s43, %[x0]\n\t" "v_fmac_f32 v57, s44, %[x0]\n\t" "v_fmac_f32 v61, s45, %[x0]\n\t"
            "s_sub_u32 %[cnt], %[cnt], 1\n\t"
            "s_cmp_lg_u32 %[cnt], 0\n\t"
            "s_cbranch_scc1 L1_%=\n\t"
            : "+{v[48:79]}"(a0), "+{v[80:111]}"(a1), [cnt] "+s"(cnt), "+{s[34:35]}"(sp)
            : [x0] "v"(x0)
            : "memory", "scc", SCLOB);
    } else if constexpr (MODE == 2) {   // 20 x (M0 write + indexed v_fmac), records resident in SGPRs
        asm volatile(
            "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
            "s_load_dwordx16 s[52:67], s[34:35], 0x40\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            "v_mov_b32 v112, %[x0]\n\t"
            "v_mov_b32 v113, %[x0]\n\t"
            "s_set_gpr_idx_on 0, 0x0\n"
            "L2_%=:\n\t"
            SET_A(112, 113)
            SET_B(113, 112)
            "s_sub_u32 %[cnt], %[cnt], 1\n\t"
            "s_cmp_lg_u32 %[cnt], 0\n\t"
            "s_cbranch_scc1 L2_%=\n\t"
            "s_mov_b32 m0, 0\n\t"
            "s_set_gpr_idx_off\n\t"
            : "+{v[48:79]}"(a0), "+{v[80:111]}"(a1), [cnt] "+s"(cnt), "+{s[34:35]}"(sp)
            : [x0] "v"(x0)
            : "memory", "scc", "m0", "v112", "v113", SCLOB);
    } else if constexpr (MODE == 3) {   // one M0 write per two v_fmac (20 fmac, 10 M0 writes per iteration)
        asm volatile(
            "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
            "s_load_dwordx16 s[52:67], s[34:35], 0x40\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            "v_mov_b32 v112, %[x0]\n\t"
            "v_mov_b32 v113, %[x0]\n\t"
            "s_set_gpr_idx_on 0, 0x0\n"
            "L3_%=:\n\t"
#define TWO(W, H) "s_mov_b32 m0, s" #H "\n\t" "v_fmac_f32 v48, s" #W ", v112\n\t" "v_fmac_f32 v80, s" #W ", v113\n\t"
            TWO(36, 46) TWO(37, 47) TWO(38, 48) TWO(39, 49) TWO(40, 50) TWO(52, 62) TWO(53, 63) TWO(54, 64) TWO(55, 65) TWO(56, 66)
            "s_sub_u32 %[cnt], %[cnt], 1\n\t"
            "s_cmp_lg_u32 %[cnt], 0\n\t"
            "s_cbranch_scc1 L3_%=\n\t"
            "s_mov_b32 m0, 0\n\t"
            "s_set_gpr_idx_off\n\t"
            : "+{v[48:79]}"(a0), "+{v[80:111]}"(a1), [cnt] "+s"(cnt), "+{s[34:35]}"(sp)
            : [x0] "v"(x0)
            : "memory", "scc", "m0", "v112", "v113", SCLOB);
    } else if constexpr (MODE == 5) {   // MODE 2 + the records streamed: one s_load_dwordx16 per 10 pairs, one set ahead
        asm volatile(
            "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
            "s_add_u32 s34, s34, 64\n\t"
            "s_addc_u32 s35, s35, 0\n\t"
            "v_mov_b32 v112, %[x0]\n\t"
            "v_mov_b32 v113, %[x0]\n\t"
            "s_set_gpr_idx_on 0, 0x0\n"
            "L5_%=:\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[52:67], s[34:35], 0x0\n\t"
            SET_A(112, 113)
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[36:51], s[34:35], 0x40\n\t"
            "s_add_u32 s34, s34, 128\n\t"
            "s_addc_u32 s35, s35, 0\n\t"
            SET_B(113, 112)
            "s_sub_u32 %[cnt], %[cnt], 1\n\t"
            "s_cmp_lg_u32 %[cnt], 0\n\t"
            "s_cbranch_scc1 L5_%=\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_mov_b32 m0, 0\n\t"
            "s_set_gpr_idx_off\n\t"
            : "+{v[48:79]}"(a0), "+{v[80:111]}"(a1), [cnt] "+s"(cnt), "+{s[34:35]}"(sp)
            : [x0] "v"(x0)
            : "memory", "scc", "m0", "v112", "v113", SCLOB);
    } else if constexpr (MODE == 6 || MODE == 7) {   // MODE 5 + X through buffer loads: one per 5 pairs, ring of 8 registers, 3 sets ahead
        // iteration = 4 sets (A, B, A, B); set i uses x[2i], x[2i+1]; during set i the loads of set i+3 are issued
#define XLOAD(V, OFF) "buffer_load_dword v" #V ", %[voff], %[rs], s" #OFF " offen\n\t"
#define XLOAD2(V, OFF) "buffer_load_dword v" #V ", %[voff], %[rs], s" #OFF " offen offset:256\n\t"
        asm volatile(
            "s_load_dwordx16 s[36:51], s[34:35], 0x0\n\t"
            "s_add_u32 s34, s34, 64\n\t"
            "s_addc_u32 s35, s35, 0\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            XLOAD(112, 51) XLOAD2(113, 51) XLOAD(114, 51) XLOAD2(115, 51) XLOAD(116, 51) XLOAD2(117, 51)
            "s_set_gpr_idx_on 0, 0x0\n"
            "L6_%=:\n\t"
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[52:67], s[34:35], 0x0\n\t"
            XLOAD(118, 51) XLOAD2(119, 51)
            "s_waitcnt vmcnt(6)\n\t"
            SET_A(112, 113)
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[36:51], s[34:35], 0x40\n\t"
            XLOAD(112, 67) XLOAD2(113, 67)
            "s_waitcnt vmcnt(6)\n\t"
            SET_B(114, 115)
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[52:67], s[34:35], 0x80\n\t"
            XLOAD(114, 51) XLOAD2(115, 51)
            "s_waitcnt vmcnt(6)\n\t"
            SET_A(116, 117)
            "s_waitcnt lgkmcnt(0)\n\t"
            "s_load_dwordx16 s[36:51], s[34:35], 0xc0\n\t"
            "s_add_u32 s34, s34, 256\n\t"
            "s_addc_u32 s35, s35, 0\n\t"
            XLOAD(116, 67) XLOAD2(117, 67)
            "s_waitcnt vmcnt(6)\n\t"
            SET_B(118, 119)
            "s_sub_u32 %[cnt], %[cnt], 1\n\t"
            "s_cmp_lg_u32 %[cnt], 0\n\t"
            "s_cbranch_scc1 L6_%=\n\t"
            "s_waitcnt vmcnt(0) lgkmcnt(0)\n\t"
            "s_mov_b32 m0, 0\n\t"
            "s_set_gpr_idx_off\n\t"
            : "+{v[48:79]}"(a0), "+{v[80:111]}"(a1), [cnt] "+s"(cnt), "+{s[34:35]}"(sp)
            : [voff] "v"(voff), [rs] "s"(rs)
            : "memory", "scc", "m0", "v112", "v113", "v114", "v115", "v116", "v117", "v118", "v119", SCLOB);
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) s += a0[i] + a1[i];
    out[blockIdx.x * blockDim.x + tid] = s;
    const unsigned long long r1 = wall_clock64();
    if (lane == 0) {
        cycles[(blockIdx.x * nw + wave) * 2] = t1 - t0;         // shader clocks
        cycles[(blockIdx.x * nw + wave) * 2 + 1] = r1 - r0;     // ticks of the constant 100 MHz counter
    }
}

template <int MODE>
void run(const char *name, int threads, uint32_t iters, double pairs_per_iter, float *out, unsigned long long *cyc, const int4 *stream,
         const float *X, uint32_t xbytes)
{
    const int blocks = 256;
    const int nw = threads / 64;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int rep = 0; rep < 3; ++rep) {
        CK(hipEventRecord(e0));
        probe<MODE><<<blocks, threads>>>(out, cyc, stream, X, iters, xbytes);
        CK(hipEventRecord(e1));
        CK(hipDeviceSynchronize());
    }
    float ms = 0; CK(hipEventElapsedTime(&ms, e0, e1));
    std::vector<unsigned long long> h((size_t)blocks * nw * 2);
    CK(hipMemcpy(h.data(), cyc, h.size() * 8, hipMemcpyDeviceToHost));
    // per wave: shader clocks and 100 MHz ticks between its first and last instruction of the loop
    std::vector<double> c, mhz;
    for (size_t w = 0; w < h.size() / 2; ++w) { c.push_back((double)h[2 * w]); mhz.push_back(h[2 * w + 1] ? h[2 * w] * 100.0 / h[2 * w + 1] : 0.0); }
    std::sort(c.begin(), c.end());
    std::sort(mhz.begin(), mhz.end());
    const double clk = c[c.size() / 2];                              // median wave
    const double pairs_simd = pairs_per_iter * iters * (nw / 4.0);    // wave-level multiply-adds per SIMD
    std::printf("%-44s waves/CU %2d  launch %7.3f ms  shader clock %4.0f MHz  clk per multiply-add: per wave %5.2f, per SIMD %5.2f  lane-FMA/clk/CU %5.1f\n",
                name, nw, ms, mhz[mhz.size() / 2], clk / (pairs_per_iter * iters), clk / pairs_simd, 4.0 * 64.0 * pairs_simd / clk);
}

int main()
{
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    std::printf("%s, %d CUs, nominal clock %d kHz; one workgroup per CU\n", prop.gcnArchName, prop.multiProcessorCount, prop.clockRate);
    float *out; unsigned long long *cyc; int4 *stream; float *X;
    const size_t stream_bytes = (size_t)256 * 16 * 65536;   // 64 KB per wave
    const uint32_t xbytes = 4096 * 256 * 4;
    CK(hipMalloc(&out, 256 * 1024 * 4)); CK(hipMalloc(&cyc, 256 * 16 * 8 * 2)); CK(hipMalloc(&stream, stream_bytes)); CK(hipMalloc(&X, xbytes));
    std::vector<uint32_t> hs(stream_bytes / 4);
    uint32_t seed = 12345;
    auto rnd = [&]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    for (size_t s = 0; s < hs.size() / 16; ++s) {
        uint32_t *d = &hs[s * 16];
        for (int k = 0; k < 10; ++k) { float w = 1.0f / (float)(1 + rnd() % 1000); d[k] = __builtin_bit_cast(uint32_t, w); }
        for (int k = 0; k < 5; ++k) d[10 + k] = (0xC000u | (rnd() % 64u)) | ((0xC000u | (rnd() % 64u)) << 16);
        d[15] = (rnd() % 4000u) * 1024u;    // byte offset of an X row segment (row * C * 4, C = 256)
    }
    CK(hipMemcpy(stream, hs.data(), stream_bytes, hipMemcpyHostToDevice));
    CK(hipMemset(X, 0, xbytes));
    // warm the clocks
    for (int i = 0; i < 20; ++i) probe<1><<<256, 1024>>>(out, cyc, stream, X, 20000, xbytes);
    CK(hipDeviceSynchronize());
    const uint32_t it = 20000;
    run<1>("static v_fmac, scalar weight", 1024, it, 20, out, cyc, stream, X, xbytes);
    run<2>("M0 write + indexed v_fmac per pair", 1024, it, 20, out, cyc, stream, X, xbytes);
    run<2>("M0 write + indexed v_fmac per pair", 768, it, 20, out, cyc, stream, X, xbytes);
    run<2>("M0 write + indexed v_fmac per pair", 512, it, 20, out, cyc, stream, X, xbytes);
    run<2>("M0 write + indexed v_fmac per pair", 256, it, 20, out, cyc, stream, X, xbytes);
    run<3>("M0 write per two v_fmac", 1024, it, 20, out, cyc, stream, X, xbytes);
    run<5>("per pair + records streamed (s_load x16)", 1024, 500, 20, out, cyc, stream, X, xbytes);
    run<5>("per pair + records streamed (s_load x16)", 768, 500, 20, out, cyc, stream, X, xbytes);
    run<5>("per pair + records streamed (s_load x16)", 512, 500, 20, out, cyc, stream, X, xbytes);
    run<6>("per pair + records + X loads", 1024, 250, 40, out, cyc, stream, X, xbytes);
    run<6>("per pair + records + X loads", 768, 250, 40, out, cyc, stream, X, xbytes);
    run<6>("per pair + records + X loads", 512, 250, 40, out, cyc, stream, X, xbytes);
    return 0;
}
