// C-ABI driver around the *reference's own* CPU kernels.  TEST INFRASTRUCTURE ONLY.
//
// This translation unit is compiled together with the reference's source files
// where they lie (see oracle/Makefile, target _ref/libsparseops_ref.so); no
// reference source is copied into this repository and the resulting library is
// not tracked by git.  It is used (a) to validate oracle.c and (b) as the CPU
// baseline of the benchmark.  It is never loaded by the shipped library.
//
// Reference entry points wrapped:
//   convert_to_ellpack / decode_from_ellpack   include/ellpack_encoder.hpp:28,32
//   ellpack_matmul (dispatcher)                include/ellpack_matmul.hpp:23-43
//   ellpack_matmul_fused<USE_MASK,FUSE_RELU>   src/ellpack_matmul.cpp:11-103
//   ellpack_matvec                             src/ellpack_matvec.cpp:20-147
//   relu/sigmoid/tanh_inplace                  src/activations.cpp:20-68
//   conv2d_patchmajor_tiled / tiled_im2col_fmajor / tiled_im2col_cmajor /
//   conv2d_rbm_fmajor_implicit                 src/layers/conv_kernels.cpp:66-470
//   build_rbm_from_ellpack                     src/layers/rbm_conv.cpp:7-73
#include <cstdint>
#include <cstring>
#include <utility>
#include <vector>

#include "ellpack_encoder.hpp"
#include "ellpack_matmul.hpp"
#include "ellpack_matvec.hpp"
#include "activations.hpp"
#include "conv_kernels.hpp"
#include "rbm_conv.hpp"

extern "C" {

void *ref_encode(const float *W, uint32_t m, uint32_t n)
{
    return new Ellpack(convert_to_ellpack(W, m, n));
}

// Build an Ellpack straight from packed arrays (for matrices generated directly
// in ELLPACK form because the dense matrix would not fit).
void *ref_from_arrays(const float *Wd, const uint32_t *idx, const uint32_t *nnz,
                      uint32_t m, uint32_t n, uint32_t r)
{
    Ellpack *E = new Ellpack(m, n, r);
    std::memcpy(E->Wd.ptr, Wd, size_t(m) * r * sizeof(float));
    std::memcpy(E->idx.data(), idx, size_t(m) * r * sizeof(uint32_t));
    std::memcpy(E->nnz.data(), nnz, size_t(m) * sizeof(uint32_t));
    return E;
}

void ref_free(void *h) { delete static_cast<Ellpack *>(h); }

void ref_dims(void *h, uint32_t *m, uint32_t *n, uint32_t *r)
{
    auto *E = static_cast<Ellpack *>(h);
    *m = E->m; *n = E->n; *r = E->r;
}

void ref_copy(void *h, float *Wd, uint32_t *idx, uint32_t *nnz)
{
    auto *E = static_cast<Ellpack *>(h);
    std::memcpy(Wd, E->Wd.ptr, size_t(E->m) * E->r * sizeof(float));
    std::memcpy(idx, E->idx.data(), size_t(E->m) * E->r * sizeof(uint32_t));
    std::memcpy(nnz, E->nnz.data(), size_t(E->m) * sizeof(uint32_t));
}

void ref_decode(void *h, float *W) { decode_from_ellpack(*static_cast<Ellpack *>(h), W); }

void ref_matmul(void *h, const float *X, uint32_t C, const float *bias, float *Y)
{
    ellpack_matmul(*static_cast<Ellpack *>(h), X, C, bias, Y);
}

void ref_matmul_fused(void *h, const float *X, uint32_t C, const float *bias, float *Y,
                      int use_mask, int fuse_relu)
{
    const Ellpack &E = *static_cast<Ellpack *>(h);
    if (use_mask) {
        if (fuse_relu) ellpack_matmul_fused<true, true>(E, X, C, bias, Y);
        else           ellpack_matmul_fused<true, false>(E, X, C, bias, Y);
    } else {
        if (fuse_relu) ellpack_matmul_fused<false, true>(E, X, C, bias, Y);
        else           ellpack_matmul_fused<false, false>(E, X, C, bias, Y);
    }
}

void ref_matvec(void *h, const float *x, const float *bias, float *y)
{
    ellpack_matvec(*static_cast<Ellpack *>(h), x, bias, y);
}

void ref_relu_inplace(float *d, size_t n) { relu_inplace(d, n); }
void ref_sigmoid_inplace(float *d, size_t n) { sigmoid_inplace(d, n); }
void ref_tanh_inplace(float *d, size_t n) { tanh_inplace(d, n); }

// geom = {Cin, Cout, kH, kW, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, H_in, W_in, H_out, W_out}
// variant: 0 patch-major tiled ([C][H][W][B]); 1 tiled im2col, Fortran (B,C,H,W);
//          2 tiled im2col, C-order NCHW; 3 RBM implicit, Fortran (B,C,H,W).
// The ConvAttr is filled the way the reference's loader fills it
// (src/sparse_onnx.cpp:394-502): weights Cout x K row-major, kmap in (cin,kh,kw)
// order with dh = kh*dil - pad, patch_indices with a one-past sentinel.
struct RefConvPlan {
    ConvAttr attr;
    std::vector<float> bias;
    int variant;
};

// Load-time part (what the reference's loader does once per layer): encode, kmap, patch_indices
// (variant 1), RBM plan (variant 3).  The bias is copied.
void *ref_conv_plan(const float *Wdense, const uint32_t *geom, const float *bias, int fuse_relu, int variant)
{
    auto *p = new RefConvPlan{ConvAttr{convert_to_ellpack(Wdense, geom[1], geom[0] * geom[2] * geom[3])}, {}, variant};
    ConvAttr &c = p->attr;
    if (bias) p->bias.assign(bias, bias + geom[1]);
    c.bias_ptr = bias ? p->bias.data() : nullptr;
    c.Cin = geom[0]; c.Cout = geom[1]; c.kH = geom[2]; c.kW = geom[3];
    c.stride_h = geom[4]; c.stride_w = geom[5];
    c.pad_h = geom[6]; c.pad_w = geom[7];
    c.dil_h = geom[8]; c.dil_w = geom[9];
    c.H_in = geom[10]; c.W_in = geom[11]; c.H_out = geom[12]; c.W_out = geom[13];
    c.fuse_relu = fuse_relu != 0;
    const uint32_t K = c.Cin * c.kH * c.kW;
    for (uint32_t ci = 0; ci < c.Cin; ++ci)
        for (uint32_t kh = 0; kh < c.kH; ++kh)
            for (uint32_t kw = 0; kw < c.kW; ++kw)
                c.kmap.push_back(KMap{ci, int32_t(kh * c.dil_h) - int32_t(c.pad_h),
                                      int32_t(kw * c.dil_w) - int32_t(c.pad_w)});
    if (variant == 1) {
        const uint32_t P = c.H_out * c.W_out;
        c.sentinel_off = size_t(c.Cin) * c.H_in * c.W_in;
        c.patch_indices.resize(size_t(K) * P);
        for (uint32_t ph = 0; ph < c.H_out; ++ph)
            for (uint32_t pw = 0; pw < c.W_out; ++pw)
                for (uint32_t k = 0; k < K; ++k) {
                    const KMap &km = c.kmap[k];
                    const int ih = int(ph * c.stride_h) + km.dh, iw = int(pw * c.stride_w) + km.dw;
                    const bool in = unsigned(ih) < c.H_in && unsigned(iw) < c.W_in;
                    c.patch_indices[size_t(ph * c.W_out + pw) * K + k] =
                        in ? (size_t(km.cin) * c.H_in + size_t(ih)) * c.W_in + size_t(iw) : c.sentinel_off;
                }
    }
    if (variant == 3) {
        c.rbm = build_rbm_from_ellpack(c.E, c.bias_ptr, 8);
        c.use_rbm = true;
    }
    return p;
}

// The per-call part: one of the reference's convolution kernels on a prepared layer.
void ref_conv_run(void *plan, const float *src, uint32_t B, float *dst)
{
    const RefConvPlan *p = static_cast<RefConvPlan *>(plan);
    switch (p->variant) {
    case 0: conv2d_patchmajor_tiled(p->attr, src, B, dst); break;
    case 1: conv2d_tiled_im2col_fmajor(p->attr, src, B, dst); break;
    case 2: conv2d_tiled_im2col_cmajor(p->attr, src, B, dst); break;
    case 3: conv2d_rbm_fmajor_implicit(p->attr, src, B, dst); break;
    default: break;
    }
}

void ref_conv_plan_free(void *plan) { delete static_cast<RefConvPlan *>(plan); }

void ref_conv(const float *Wdense, const uint32_t *geom, const float *bias, int fuse_relu,
              int variant, const float *src, uint32_t B, float *dst)
{
    void *p = ref_conv_plan(Wdense, geom, bias, fuse_relu, variant);
    ref_conv_run(p, src, B, dst);
    ref_conv_plan_free(p);
}

// build_rbm_from_ellpack on the handle's matrix, flattened: sizes = {blocks, union columns, pairs};
// block_union[b] = union columns before block b, colptr made absolute over all blocks.
void ref_rbm_sizes(void *h, uint32_t Ct_max, uint32_t *sizes)
{
    const RBMPlan P = build_rbm_from_ellpack(*static_cast<Ellpack *>(h), nullptr, Ct_max);
    sizes[0] = uint32_t(P.blocks.size());
    sizes[1] = sizes[2] = 0;
    for (const RBMBlock &b : P.blocks) { sizes[1] += uint32_t(b.krel.size()); sizes[2] += uint32_t(b.pairs.size()); }
}

void ref_rbm_copy(void *h, uint32_t Ct_max, uint32_t *block_union, uint32_t *krel, uint32_t *colptr,
                  uint16_t *pair_row, float *pair_w)
{
    const RBMPlan P = build_rbm_from_ellpack(*static_cast<Ellpack *>(h), nullptr, Ct_max);
    uint32_t u = 0, p = 0;
    block_union[0] = 0;
    colptr[0] = 0;
    for (size_t b = 0; b < P.blocks.size(); ++b) {
        const RBMBlock &B = P.blocks[b];
        for (size_t k = 0; k < B.krel.size(); ++k) {
            krel[u] = B.krel[k];
            colptr[u + 1] = p + B.colptr[k + 1];
            ++u;
        }
        for (const RBMColPair &q : B.pairs) { pair_row[p] = q.row; pair_w[p] = q.w; ++p; }
        block_union[b + 1] = u;
    }
}

} // extern "C"
