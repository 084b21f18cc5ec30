/*
 * CPU oracle for the ELLPACK compute path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's CPU kernels so
 * that the HIP kernels can be checked against it.  Nothing shipped (the HIP
 * library, the host C++ layer, the pybind11 module) links, loads or calls it; only
 * the test-suite, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function names the reference file:line it follows.  Pinning status
 * (what independent evidence fixes each function) is listed here and checked in
 * tests/test_oracle_*.py:
 *
 *   orc_ellpack_count/pack  reference known-answer 4x4 (tests/unit/test_ellpack_encoder.py:51-77),
 *                           numpy closed forms, decode(encode(W)) == W, compiled reference
 *   orc_ellpack_decode      round trip, compiled reference
 *   orc_matmul              fp64 dense W@X+bias, linearity/special cases, compiled reference (bit-exact)
 *   orc_matvec              fp64 dense W@x+bias, compiled reference AVX-512 path (bit-exact)
 *   orc_act                 numpy maximum / 1/(1+exp(-x)) / tanh in fp64, compiled reference in-place kernels
 *   orc_conv2d_pf           7-loop brute force, torch conv2d, 1x1 == matmul, delta kernel == shift,
 *                           compiled reference conv2d_patchmajor_tiled (bit-exact up to the sign of zero)
 *   orc_rbm_build           hand-written known answer, (column,row)-sorted numpy triples, decode(RBM) == W,
 *                           compiled reference build_rbm_from_ellpack (identical arrays)
 *   orc_conv2d_rbm_pf       orc_conv2d_pf (same bits: per-channel order is unchanged), compiled reference
 *                           conv2d_rbm_fmajor_implicit, 1x1 == orc_matmul
 *   orc_maxpool_pf          numpy brute force, torch max_pool2d
 *   orc_gap_pf              numpy mean (tolerance), explicit (h,w)-ordered fp32 sum times reciprocal
 *   orc_add                 numpy
 *
 * Build: see oracle/Makefile (gcc -O3 -march=x86-64-v3 -ffp-contract=off -fopenmp).
 * fmaf() must compile to a hardware FMA (x86-64-v3 guarantees it) so that the
 * in-order accumulation is the same correctly rounded sequence the reference's
 * _mm512_fmadd_ps loop produces.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { ORC_ACT_NONE = 0, ORC_ACT_RELU = 1, ORC_ACT_SIGMOID = 2, ORC_ACT_TANH = 3 };

/* ------------------------------------------------------------------ encoder */

/* Pass 1 of convert_to_ellpack (src/ellpack_encoder.cpp:8-17): per-row count of
 * entries with v != 0.0f (so -0.0f is dropped and NaN is kept); returns r = max. */
uint32_t orc_ellpack_count(const float *W, uint32_t m, uint32_t n, uint32_t *nnz)
{
    uint32_t r = 0;
    for (uint32_t i = 0; i < m; ++i) {
        const float *row = W + (size_t)i * n;
        uint32_t cnt = 0;
        for (uint32_t j = 0; j < n; ++j)
            if (row[j] != 0.0f) ++cnt;
        nnz[i] = cnt;
        if (cnt > r) r = cnt;
    }
    return r;
}

/* Pass 2 (src/ellpack_encoder.cpp:24-41): Wd zero-filled, idx zero-filled (the
 * reference's std::vector value-initialises, include/ellpack_encoder.hpp:17-19),
 * then values and columns packed in ascending column order. */
void orc_ellpack_pack(const float *W, uint32_t m, uint32_t n, uint32_t r,
                      float *Wd, uint32_t *idx)
{
    memset(Wd, 0, (size_t)m * r * sizeof(float));
    memset(idx, 0, (size_t)m * r * sizeof(uint32_t));
    for (uint32_t i = 0; i < m; ++i) {
        const float *row = W + (size_t)i * n;
        size_t base = (size_t)i * r;
        uint32_t pos = 0;
        for (uint32_t j = 0; j < n; ++j) {
            float v = row[j];
            if (v != 0.0f) {
                Wd[base + pos] = v;
                idx[base + pos] = j;
                ++pos;
            }
        }
    }
}

/* decode_from_ellpack (src/ellpack_encoder.cpp:46-60). */
void orc_ellpack_decode(const float *Wd, const uint32_t *idx, const uint32_t *nnz,
                        uint32_t m, uint32_t n, uint32_t r, float *W)
{
    memset(W, 0, (size_t)m * n * sizeof(float));
    for (uint32_t i = 0; i < m; ++i)
        for (uint32_t j = 0; j < nnz[i]; ++j)
            W[(size_t)i * n + idx[(size_t)i * r + j]] = Wd[(size_t)i * r + j];
}

/* ------------------------------------------------------------- activations */

/* src/layers/activation.cpp:17-20 (v > 0 ? v : 0), :38-40 (1/(1+exp(-v)) in
 * float), :58-60 (tanh in float). */
static inline float orc_act1(float v, int act)
{
    switch (act) {
    case ORC_ACT_RELU:    return v > 0.0f ? v : 0.0f;
    case ORC_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
    case ORC_ACT_TANH:    return tanhf(v);
    default:              return v;
    }
}

void orc_act(const float *src, size_t len, int act, float *dst)
{
    for (size_t i = 0; i < len; ++i) dst[i] = orc_act1(src[i], act);
}

/* ------------------------------------------------------------------ matmul */

/* ellpack_matmul_fused (src/ellpack_matmul.cpp:11-92): every output element
 * starts from bias[i] (or 0) and receives one hardware FMA per stored nonzero of
 * row i in ascending slot order (:56-66); optional ReLU afterwards (:68-70).
 * The reference only fuses ReLU; act = SIGMOID/TANH here means "then apply the
 * separate activation layer" (src/layers/activation.cpp), which is what a fused
 * epilogue must equal.  Column tiling (16 wide in the reference) does not change
 * any element's arithmetic, so the tile width here is free. */
void orc_matmul(const float *Wd, const uint32_t *idx, const uint32_t *nnz,
                uint32_t m, uint32_t n, uint32_t r,
                const float *X, uint32_t C, const float *bias, int act, float *Y)
{
    (void)n;
#pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < m; ++i) {
        float *yrow = Y + (size_t)i * C;
        const size_t base = (size_t)i * r;
        const uint32_t cnt = nnz[i];
        const float b = bias ? bias[i] : 0.0f;
        uint32_t cb = 0;
        for (; cb + 32 <= C; cb += 32) {
            float acc[32];
            for (int l = 0; l < 32; ++l) acc[l] = b;
            for (uint32_t j = 0; j < cnt; ++j) {
                const float w = Wd[base + j];
                const float *x = X + (size_t)idx[base + j] * C + cb;
#pragma omp simd
                for (int l = 0; l < 32; ++l) acc[l] = fmaf(w, x[l], acc[l]);
            }
            for (int l = 0; l < 32; ++l) yrow[cb + l] = orc_act1(acc[l], act);
        }
        for (; cb < C; ++cb) {
            float a = b;
            for (uint32_t j = 0; j < cnt; ++j)
                a = fmaf(Wd[base + j], X[(size_t)idx[base + j] * C + cb], a);
            yrow[cb] = orc_act1(a, act);
        }
    }
}

/* Same arithmetic with no tiling at all: one scalar fmaf chain per element.
 * Exists so a test can show that the tiled loop above did not change a bit. */
void orc_matmul_scalar(const float *Wd, const uint32_t *idx, const uint32_t *nnz,
                       uint32_t m, uint32_t n, uint32_t r,
                       const float *X, uint32_t C, const float *bias, int act, float *Y)
{
    (void)n;
    for (uint32_t i = 0; i < m; ++i)
        for (uint32_t c = 0; c < C; ++c) {
            volatile float a = bias ? bias[i] : 0.0f;
            for (uint32_t j = 0; j < nnz[i]; ++j)
                a = fmaf(Wd[(size_t)i * r + j], X[(size_t)idx[(size_t)i * r + j] * C + c], a);
            Y[(size_t)i * C + c] = orc_act1(a, act);
        }
}

/* ------------------------------------------------------------------ matvec */

/* ellpack_matvec, AVX-512 path (src/ellpack_matvec.cpp:43-100): 16 interleaved
 * partial sums over the first nnz[i] slots (lane l takes slots l, l+16, ...; one
 * FMA per slot, :72-85, the masked tail adds fma(0,0,acc) = acc to idle lanes),
 * then the tree 16->8->4->2->1 (:88-96: lo8+hi8, lo4+hi4, two hadds), then
 * y[i] = bias[i] + acc (:30-34, :99). */
void orc_matvec(const float *Wd, const uint32_t *idx, const uint32_t *nnz,
                uint32_t m, uint32_t n, uint32_t r,
                const float *x, const float *bias, float *y)
{
    (void)n;
#pragma omp parallel for schedule(static)
    for (uint32_t i = 0; i < m; ++i) {
        const size_t base = (size_t)i * r;
        const uint32_t cnt = nnz[i];
        float acc[16];
        for (int l = 0; l < 16; ++l) acc[l] = 0.0f;
        for (uint32_t j = 0; j < cnt; ++j)
            acc[j & 15] = fmaf(Wd[base + j], x[idx[base + j]], acc[j & 15]);
        float s8[8], s4[4];
        for (int l = 0; l < 8; ++l) s8[l] = acc[l] + acc[l + 8];
        for (int l = 0; l < 4; ++l) s4[l] = s8[l] + s8[l + 4];
        const float h0 = s4[0] + s4[1];
        const float h1 = s4[2] + s4[3];
        const float dot = h0 + h1;
        y[i] = (bias ? bias[i] : 0.0f) + dot;
    }
}

/* -------------------------------------------------------------------- conv */

/* Geometry of one Conv node as the loader derives it (src/sparse_onnx.cpp:408-451):
 * only the begin pads are used, H_out = (H + 2p - (d(k-1)+1))/s + 1, and column k
 * of the Cout x K weight matrix is (cin, kh, kw) = (k / (kH*kW), (k / kW) % kH, k % kW). */
typedef struct {
    uint32_t Cin, Cout, kH, kW;
    uint32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
    uint32_t H_in, W_in, H_out, W_out;
} orc_conv_geom;

/* Sparse convolution by implicit im2col, the arithmetic of
 * conv2d_implicit_im2col_fmajor (src/layers/conv.cpp:44-107): accumulator starts
 * at bias[co], one FMA per stored nonzero in ascending slot order, taps that fall
 * outside the image are skipped (:66), optional ReLU (:77).  Activations use the
 * patch-major layout [C][H][W][B] (batch innermost) that the reference's
 * applyConv feeds conv2d_patchmajor_tiled (src/layers/conv_kernels.cpp:342-347);
 * the tiled kernel performs fma(w, 0, acc) for padded taps instead of skipping
 * them, which differs at most in the sign of a zero result. */
void orc_conv2d_pf(const float *Wd, const uint32_t *idx, const uint32_t *nnz, uint32_t r,
                   const orc_conv_geom *g, const float *X, uint32_t B,
                   const float *bias, int act, float *Y)
{
    const uint32_t H = g->H_in, W = g->W_in, Ho = g->H_out, Wo = g->W_out;
    const uint32_t kHW = g->kH * g->kW;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t co = 0; co < g->Cout; ++co)
        for (uint32_t ho = 0; ho < Ho; ++ho)
            for (uint32_t wo = 0; wo < Wo; ++wo) {
                float *yp = Y + (((size_t)co * Ho + ho) * Wo + wo) * B;
                const float b0 = bias ? bias[co] : 0.0f;
                for (uint32_t b = 0; b < B; ++b) yp[b] = b0;
                for (uint32_t j = 0; j < nnz[co]; ++j) {
                    const float w = Wd[(size_t)co * r + j];
                    const uint32_t k = idx[(size_t)co * r + j];
                    const uint32_t cin = k / kHW, kh = (k / g->kW) % g->kH, kw = k % g->kW;
                    const int32_t hin = (int32_t)(ho * g->stride_h) + (int32_t)(kh * g->dil_h) - (int32_t)g->pad_h;
                    const int32_t win = (int32_t)(wo * g->stride_w) + (int32_t)(kw * g->dil_w) - (int32_t)g->pad_w;
                    if ((uint32_t)hin >= H || (uint32_t)win >= W) continue;
                    const float *xp = X + (((size_t)cin * H + (uint32_t)hin) * W + (uint32_t)win) * B;
                    for (uint32_t b = 0; b < B; ++b) yp[b] = fmaf(w, xp[b], yp[b]);
                }
                for (uint32_t b = 0; b < B; ++b) yp[b] = orc_act1(yp[b], act);
            }
}

/* ------------------------------------------------ row-block-merged format */

typedef struct { uint32_t k; uint32_t r; float w; } orc_trip;

static int orc_trip_cmp(const void *a, const void *b)
{
    const orc_trip *x = (const orc_trip *)a, *y = (const orc_trip *)b;
    if (x->k != y->k) return x->k < y->k ? -1 : 1;
    return x->r < y->r ? -1 : (x->r > y->r ? 1 : 0);
}

/* build_rbm_from_ellpack (src/layers/rbm_conv.cpp:7-73), flattened: per block of Ct_max rows the
 * (column, row in block, weight) triples of the rows' first nnz slots (:23-31) are ordered by
 * (column, row) (:38-39) and cut into runs of equal column, one union column per run (:41-63).
 * block_union[b] = union columns before block b; colptr is absolute over all blocks.  Called
 * twice: with krel == NULL it only counts.  Returns via sizes = {union columns, pairs}. */
void orc_rbm_build(const float *Wd, const uint32_t *idx, const uint32_t *nnz, uint32_t m, uint32_t r,
                   uint32_t Ct_max, uint32_t *block_union, uint32_t *krel, uint32_t *colptr,
                   uint16_t *pair_row, float *pair_w, uint64_t *sizes)
{
    orc_trip *all = (orc_trip *)malloc(sizeof(orc_trip) * ((size_t)Ct_max * r + 1));
    uint64_t U = 0, P = 0;
    uint32_t b = 0;
    if (block_union) block_union[0] = 0;
    if (krel) colptr[0] = 0;
    for (uint32_t M0 = 0; M0 < m; M0 += Ct_max, ++b) {
        const uint32_t Ct = m - M0 < Ct_max ? m - M0 : Ct_max;
        size_t cnt = 0;
        for (uint32_t rr = 0; rr < Ct; ++rr) {
            const size_t base = (size_t)(M0 + rr) * r;
            for (uint32_t j = 0; j < nnz[M0 + rr]; ++j) {
                all[cnt].k = idx[base + j];
                all[cnt].r = rr;
                all[cnt].w = Wd[base + j];
                ++cnt;
            }
        }
        qsort(all, cnt, sizeof(orc_trip), orc_trip_cmp);
        for (size_t t = 0; t < cnt; ++t) {
            if (t == 0 || all[t].k != all[t - 1].k) {
                if (krel) krel[U] = all[t].k;
                ++U;
            }
            if (krel) {
                pair_row[P] = (uint16_t)all[t].r;
                pair_w[P] = all[t].w;
                colptr[U] = (uint32_t)(P + 1);
            }
            ++P;
        }
        if (block_union) block_union[b + 1] = (uint32_t)U;
    }
    free(all);
    sizes[0] = U;
    sizes[1] = P;
}

/* conv2d_rbm_fmajor_implicit (src/layers/conv_kernels.cpp:66-147) on the [C][H][W][B] layout: per
 * output pixel and block the accumulators start at the bias (:100-104); the block's union columns
 * are walked once in order, a tap outside the image is skipped (:112-114), its input vector is
 * multiply-added (fused) into every row that has a pair at that column (:118-123); optional ReLU
 * (:126-130; the other activations are this build's epilogues).  Blocks of at most 64 rows. */
void orc_conv2d_rbm_pf(const uint32_t *block_union, const uint32_t *krel, const uint32_t *colptr,
                       const uint16_t *pair_row, const float *pair_w, uint32_t Ct_max,
                       const orc_conv_geom *g, const float *X, uint32_t B,
                       const float *bias, int act, float *Y)
{
    const uint32_t H = g->H_in, W = g->W_in, Ho = g->H_out, Wo = g->W_out;
    const uint32_t kHW = g->kH * g->kW;
    const uint32_t nblocks = (g->Cout + Ct_max - 1) / Ct_max;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t ho = 0; ho < Ho; ++ho)
        for (uint32_t wo = 0; wo < Wo; ++wo)
            for (uint32_t blk = 0; blk < nblocks; ++blk) {
                const uint32_t M0 = blk * Ct_max;
                const uint32_t Ct = g->Cout - M0 < Ct_max ? g->Cout - M0 : Ct_max;
                float *yp[64];
                for (uint32_t rr = 0; rr < Ct; ++rr) {
                    yp[rr] = Y + (((size_t)(M0 + rr) * Ho + ho) * Wo + wo) * B;
                    const float b0 = bias ? bias[M0 + rr] : 0.0f;
                    for (uint32_t b = 0; b < B; ++b) yp[rr][b] = b0;
                }
                for (uint32_t u = block_union[blk]; u < block_union[blk + 1]; ++u) {
                    const uint32_t k = krel[u];
                    const uint32_t cin = k / kHW, kh = (k / g->kW) % g->kH, kw = k % g->kW;
                    const int32_t hin = (int32_t)(ho * g->stride_h) + (int32_t)(kh * g->dil_h) - (int32_t)g->pad_h;
                    const int32_t win = (int32_t)(wo * g->stride_w) + (int32_t)(kw * g->dil_w) - (int32_t)g->pad_w;
                    if ((uint32_t)hin >= H || (uint32_t)win >= W) continue;
                    const float *xp = X + (((size_t)cin * H + (uint32_t)hin) * W + (uint32_t)win) * B;
                    for (uint32_t p = colptr[u]; p < colptr[u + 1]; ++p) {
                        float *y = yp[pair_row[p]];
                        const float w = pair_w[p];
                        for (uint32_t b = 0; b < B; ++b) y[b] = fmaf(w, xp[b], y[b]);
                    }
                }
                for (uint32_t rr = 0; rr < Ct; ++rr)
                    for (uint32_t b = 0; b < B; ++b) yp[rr][b] = orc_act1(yp[rr][b], act);
            }
}

/* ------------------------------------------------------- pool / add layers */

typedef struct {
    uint32_t C, H, W, H_out, W_out;
    int32_t kH, kW, sH, sW, padH0, padW0;
} orc_pool_geom;

/* applyMaxPool (src/layers/pool.cpp:28-101): -inf start, window taps outside the
 * image skipped (:62-66), max.  Layout [C][H][W][B]. */
void orc_maxpool_pf(const orc_pool_geom *p, const float *X, uint32_t B, float *Y)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t c = 0; c < p->C; ++c)
        for (uint32_t ho = 0; ho < p->H_out; ++ho)
            for (uint32_t wo = 0; wo < p->W_out; ++wo) {
                float *yp = Y + (((size_t)c * p->H_out + ho) * p->W_out + wo) * B;
                for (uint32_t b = 0; b < B; ++b) yp[b] = -INFINITY;
                for (int32_t kh = 0; kh < p->kH; ++kh) {
                    const int32_t hin = (int32_t)ho * p->sH - p->padH0 + kh;
                    if ((uint32_t)hin >= p->H) continue;
                    for (int32_t kw = 0; kw < p->kW; ++kw) {
                        const int32_t win = (int32_t)wo * p->sW - p->padW0 + kw;
                        if ((uint32_t)win >= p->W) continue;
                        const float *xp = X + (((size_t)c * p->H + (uint32_t)hin) * p->W + (uint32_t)win) * B;
                        for (uint32_t b = 0; b < B; ++b) yp[b] = xp[b] > yp[b] ? xp[b] : yp[b];
                    }
                }
            }
}

/* applyGlobalAveragePool (src/layers/pool.cpp:103-154): fp32 running sum over
 * h (outer) then w (inner) (:129-135), multiplied by 1.0f/float(H*W) (:118,:138).
 * In [C][H][W][B] out [C][B]. */
void orc_gap_pf(uint32_t C, uint32_t H, uint32_t W, const float *X, uint32_t B, float *Y)
{
    const float scale = 1.0f / (float)(H * W);
#pragma omp parallel for schedule(static)
    for (uint32_t c = 0; c < C; ++c)
        for (uint32_t b = 0; b < B; ++b) {
            float s = 0.0f;
            for (uint32_t h = 0; h < H; ++h)
                for (uint32_t w = 0; w < W; ++w)
                    s = s + X[(((size_t)c * H + h) * W + w) * B + b];
            Y[(size_t)c * B + b] = s * scale;
        }
}

/* applyAdd (src/layers/add.cpp:9-76): D = A + B elementwise, no broadcasting. */
void orc_add(const float *A, const float *Bv, size_t len, float *D)
{
    for (size_t i = 0; i < len; ++i) D[i] = A[i] + Bv[i];
}

/* ------------------------------------------------------------------- misc */

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
