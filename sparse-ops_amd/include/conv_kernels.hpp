// Host-pointer convolution entry points with the reference's names and signatures
// (include/conv_kernels.hpp:8-36), executed on the GPU.  All four compute the same operator --
// Conv2d as the reference's implicit-im2col kernel defines it (src/layers/conv.cpp:16-108): begin
// pads, stride, dilation, group 1, bias, optional fused ReLU, one fused multiply-add per stored
// nonzero in ascending slot order -- and differ only in the layout of `src` / `dst`:
//
//   conv2d_patchmajor_tiled      [C][H][W][B]              (the device layout: no conversion)
//   conv2d_rbm_fmajor_implicit   Fortran (B,C,H,W): element (b,c,h,w) at b + B*(c + C*(h + H*w))
//   conv2d_tiled_im2col_fmajor   the same Fortran layout
//   conv2d_tiled_im2col_cmajor   C-order (B,C,H,W)
//
// The last three convert on the GPU on the way in and out (a 2-D transpose for the C-order layout, a
// reversal of the three outer axes for the Fortran one).  The first call on a ConvAttr uploads the
// weights' device copy (cached on c.E), builds the convolution plan and, with c.use_rbm set and c.rbm
// built (build_rbm_from_ellpack), the row-block-merged streams, and keeps them with the staging
// buffers on c.device; a repeated call with the same batch only copies src in, launches, and copies
// dst out -- it allocates nothing.  Convenience entry points for callers that drive single layers;
// SparseOnnxModel keeps activations resident as well.  The result has the same bits with or without
// the row-block-merged kernel.
// (For stride_w != 1 the reference's patch-major and C-major variants advance the input column by 1
// instead of stride_w, src/layers/conv_kernels.cpp:436-447, 304-313; these compute the convolution.)
// Throw std::runtime_error when no HIP device is usable or the geometry is inconsistent.
#pragma once

#include <cstdint>

#include "layer_attrs.hpp"

void conv2d_rbm_fmajor_implicit(const ConvAttr &c, const float *src, uint32_t B, float *dst);
void conv2d_tiled_im2col_fmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst);
void conv2d_tiled_im2col_cmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst);
void conv2d_patchmajor_tiled(const ConvAttr &c, const float *src_pf, uint32_t B, float *dst_pf);
