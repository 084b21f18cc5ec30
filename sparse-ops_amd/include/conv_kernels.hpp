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
// The last three convert on the host on the way in and out.  Each call uploads the weights' device
// copy if it is not resident yet (cached on c.E), builds a convolution plan, copies src in and dst
// out: convenience entry points for callers that drive single layers; SparseOnnxModel keeps plans
// and activations resident.  With c.use_rbm set and c.rbm built (build_rbm_from_ellpack) the
// row-block-merged kernel is attached to the plan; the result has the same bits either way.
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
