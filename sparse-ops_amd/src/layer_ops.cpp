// Host-pointer layer entry points with the reference's signatures (activations.hpp,
// conv_kernels.hpp), executed on the GPU through the C ABI.
#include "activations.hpp"
#include "conv_kernels.hpp"

#include <vector>

#include "device.hpp"

namespace {

using namespace sparseops;

void act_inplace(int act, float *data, std::size_t len)
{
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (len == 0) return;
    DeviceBuffer buf(len * sizeof(float));
    check(so_h2d(ctx, buf.get(), data, len * sizeof(float)), "so_h2d");
    check(so_act(ctx, act, buf.f32(), len, buf.f32()), "so_act");
    check(so_d2h(ctx, data, buf.get(), len * sizeof(float)), "so_d2h");
}

bool rows_ascend(const Ellpack &E)
{
    for (uint32_t i = 0; i < E.m; ++i)
        for (uint32_t k = 1; k < E.nnz[i]; ++k)
            if (E.idx[std::size_t(i) * E.r + k] <= E.idx[std::size_t(i) * E.r + k - 1]) return false;
    return true;
}

// The convolution on [C][H][W][B] host buffers.
void conv_pf(const ConvAttr &c, const float *src_pf, uint32_t B, float *dst_pf)
{
    if (c.group != 1) throw std::runtime_error("Only group=1 Conv supported");      // src/sparse_onnx.cpp:416
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    const std::size_t in = std::size_t(c.Cin) * c.H_in * c.W_in * B, out = std::size_t(c.Cout) * c.H_out * c.W_out * B;
    if (out == 0) return;
    so_conv_geom g{c.Cin, c.Cout, c.kH, c.kW, c.stride_h, c.stride_w, c.pad_h, c.pad_w, c.dil_h, c.dil_w, c.H_in, c.W_in, c.H_out, c.W_out};
    const so_ellpack *dE = mirror(c.E, SO_LAYOUT_ROW);
    so_conv_plan *plan = nullptr;
    check(so_conv_plan_create(ctx, dE, &g, &plan), "so_conv_plan_create");
    so_rbm *rbm = nullptr;
    struct Cleanup {
        so_ctx *ctx; so_conv_plan *&plan; so_rbm *&rbm;
        ~Cleanup() { if (plan) (void)so_conv_plan_free(ctx, plan); if (rbm) (void)so_rbm_free(ctx, rbm); }
    } cleanup{ctx, plan, rbm};
    if (B % 4 == 0) check(so_conv_plan_tune(ctx, plan, B), "so_conv_plan_tune");
    // The row-block-merged kernel takes blocks of at most 8 rows whose pairs ascend (what build_rbm_from_ellpack
    // makes of rows with ascending columns); any other plan -- the reference's kernel allows blocks of up to 16
    // rows, and a hand-filled matrix may have unordered rows -- runs on the per-row kernels: same result, same bits.
    if (c.use_rbm && !c.rbm.blocks.empty() && c.rbm.Ct_max <= 8 && rows_ascend(c.E)) {
        rbm = upload_rbm(c.rbm);
        check(so_conv_plan_set_rbm(ctx, plan, rbm), "so_conv_plan_set_rbm");
    }
    DeviceBuffer dX(in * sizeof(float)), dY(out * sizeof(float)), dB;
    check(so_h2d(ctx, dX.get(), src_pf, in * sizeof(float)), "so_h2d(src)");
    if (c.bias_ptr) {
        dB.reserve(std::size_t(c.Cout) * sizeof(float));
        check(so_h2d(ctx, dB.get(), c.bias_ptr, std::size_t(c.Cout) * sizeof(float)), "so_h2d(bias)");
    }
    check(so_conv2d(ctx, plan, dX.f32(), B, c.bias_ptr ? dB.f32() : nullptr, dY.f32(), c.fuse_relu ? SO_ACT_RELU : SO_ACT_NONE), "so_conv2d");
    check(so_d2h(ctx, dst_pf, dY.get(), out * sizeof(float)), "so_d2h(dst)");
}

// Element (b, ch, h, w) of a (B, C, H, W) tensor in the three layouts.
inline std::size_t at_pf(uint32_t b, uint32_t ch, uint32_t h, uint32_t w, uint32_t B, uint32_t, uint32_t H, uint32_t W)
{
    return ((std::size_t(ch) * H + h) * W + w) * B + b;
}
inline std::size_t at_fortran(uint32_t b, uint32_t ch, uint32_t h, uint32_t w, uint32_t B, uint32_t C, uint32_t H, uint32_t)
{
    return b + std::size_t(B) * (ch + std::size_t(C) * (h + std::size_t(H) * w));
}
inline std::size_t at_c(uint32_t b, uint32_t ch, uint32_t h, uint32_t w, uint32_t, uint32_t C, uint32_t H, uint32_t W)
{
    return ((std::size_t(b) * C + ch) * H + h) * W + w;
}

template <typename At>
void conv_converted(const ConvAttr &c, const float *src, uint32_t B, float *dst, At at)
{
    std::vector<float> in(std::size_t(c.Cin) * c.H_in * c.W_in * B), out(std::size_t(c.Cout) * c.H_out * c.W_out * B);
    for (uint32_t ch = 0; ch < c.Cin; ++ch)
        for (uint32_t h = 0; h < c.H_in; ++h)
            for (uint32_t w = 0; w < c.W_in; ++w)
                for (uint32_t b = 0; b < B; ++b)
                    in[at_pf(b, ch, h, w, B, c.Cin, c.H_in, c.W_in)] = src[at(b, ch, h, w, B, c.Cin, c.H_in, c.W_in)];
    conv_pf(c, in.data(), B, out.data());
    for (uint32_t ch = 0; ch < c.Cout; ++ch)
        for (uint32_t h = 0; h < c.H_out; ++h)
            for (uint32_t w = 0; w < c.W_out; ++w)
                for (uint32_t b = 0; b < B; ++b)
                    dst[at(b, ch, h, w, B, c.Cout, c.H_out, c.W_out)] = out[at_pf(b, ch, h, w, B, c.Cout, c.H_out, c.W_out)];
}

} // namespace

void relu_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_RELU, data, len); }
void sigmoid_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_SIGMOID, data, len); }
void tanh_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_TANH, data, len); }

void conv2d_patchmajor_tiled(const ConvAttr &c, const float *src_pf, uint32_t B, float *dst_pf) { conv_pf(c, src_pf, B, dst_pf); }
void conv2d_rbm_fmajor_implicit(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_converted(c, src, B, dst, at_fortran); }
void conv2d_tiled_im2col_fmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_converted(c, src, B, dst, at_fortran); }
void conv2d_tiled_im2col_cmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_converted(c, src, B, dst, at_c); }
