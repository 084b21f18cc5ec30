// Host-pointer layer entry points with the reference's signatures (activations.hpp,
// conv_kernels.hpp), executed on the GPU through the C ABI.
#include "activations.hpp"
#include "conv_kernels.hpp"

#include <algorithm>
#include <memory>
#include <vector>

#include "device.hpp"

namespace {

using namespace sparseops;

void act_inplace(int act, float *data, std::size_t len)
{
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (len == 0) return;
    static DeviceBuffer &buf = *new DeviceBuffer();      // grow-only, lives as long as the context (never destroyed)
    buf.reserve(len * sizeof(float));
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

// The layer's device-side state, built on the first call and kept on the ConvAttr.
ConvMirror &conv_mirror(const ConvAttr &c, uint32_t B)
{
    so_ctx *ctx = context();
    const so_ellpack *dE = mirror(c.E, SO_LAYOUT_ROW);
    const uint32_t geom[14] = {c.Cin, c.Cout, c.kH, c.kW, c.stride_h, c.stride_w, c.pad_h, c.pad_w,
                               c.dil_h, c.dil_w, c.H_in, c.W_in, c.H_out, c.W_out};
    const bool want_rbm = c.use_rbm && !c.rbm.blocks.empty();
    ConvMirror *M = c.device.get();
    if (!M || M->ellpack != c.E.device.get() || M->with_rbm != want_rbm || !std::equal(geom, geom + 14, M->geom)) {
        auto fresh = std::make_shared<ConvMirror>();
        so_conv_geom g{c.Cin, c.Cout, c.kH, c.kW, c.stride_h, c.stride_w, c.pad_h, c.pad_w, c.dil_h, c.dil_w,
                       c.H_in, c.W_in, c.H_out, c.W_out};
        check(so_conv_plan_create(ctx, dE, &g, &fresh->plan), "so_conv_plan_create");
        // The row-block-merged kernel takes blocks of at most 8 rows whose pairs ascend (what build_rbm_from_ellpack
        // makes of rows with ascending columns); any other plan -- the reference's kernel allows blocks of up to 16
        // rows, and a hand-filled matrix may have unordered rows -- runs on the per-row kernels: same result, same bits.
        if (want_rbm && c.rbm.Ct_max <= 8 && rows_ascend(c.E)) {
            fresh->rbm = upload_rbm(c.rbm);
            check(so_conv_plan_set_rbm(ctx, fresh->plan, fresh->rbm), "so_conv_plan_set_rbm");
        }
        std::copy(geom, geom + 14, fresh->geom);
        fresh->ellpack = c.E.device.get();
        fresh->with_rbm = want_rbm;
        c.device = std::move(fresh);
        M = c.device.get();
    }
    if (B % 4 == 0 && M->tuned_batch != B) {
        check(so_conv_plan_tune(ctx, M->plan, B), "so_conv_plan_tune");
        M->tuned_batch = B;
    }
    return *M;
}

enum class Layout { PatchMajor, Fortran, COrder };

// The convolution on host buffers in one of the three layouts; conversions run on the device.
void conv_any(const ConvAttr &c, const float *src, uint32_t B, float *dst, Layout layout)
{
    if (c.group != 1) throw std::runtime_error("Only group=1 Conv supported");      // src/sparse_onnx.cpp:416
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    const std::size_t in = std::size_t(c.Cin) * c.H_in * c.W_in * B, out = std::size_t(c.Cout) * c.H_out * c.W_out * B;
    if (out == 0) return;
    ConvMirror &M = conv_mirror(c, B);
    M.in.reserve(in * sizeof(float));
    M.out.reserve(out * sizeof(float));
    if (layout != Layout::PatchMajor) M.staged.reserve(std::max(in, out) * sizeof(float));
    if (layout == Layout::PatchMajor) {
        check(so_h2d(ctx, M.in.get(), src, in * sizeof(float)), "so_h2d(src)");
    } else {
        check(so_h2d(ctx, M.staged.get(), src, in * sizeof(float)), "so_h2d(src)");
        if (layout == Layout::COrder)        // (B, C*H*W) row-major -> [C*H*W][B]
            check(so_transpose(ctx, M.staged.f32(), B, uint32_t(in / B), M.in.f32()), "so_transpose");
        else                                 // Fortran (B,C,H,W) is [W][H][C][B] in memory
            check(so_reverse_axes3(ctx, M.staged.f32(), c.W_in, c.H_in, c.Cin, B, M.in.f32()), "so_reverse_axes3");
    }
    if (c.bias_ptr) {
        M.bias.reserve(std::size_t(c.Cout) * sizeof(float));
        check(so_h2d(ctx, M.bias.get(), c.bias_ptr, std::size_t(c.Cout) * sizeof(float)), "so_h2d(bias)");
    }
    check(so_conv2d(ctx, M.plan, M.in.f32(), B, c.bias_ptr ? M.bias.f32() : nullptr, M.out.f32(),
                    c.fuse_relu ? SO_ACT_RELU : SO_ACT_NONE), "so_conv2d");
    if (layout == Layout::PatchMajor) {
        check(so_d2h(ctx, dst, M.out.get(), out * sizeof(float)), "so_d2h(dst)");
    } else {
        if (layout == Layout::COrder)
            check(so_transpose(ctx, M.out.f32(), uint32_t(out / B), B, M.staged.f32()), "so_transpose");
        else
            check(so_reverse_axes3(ctx, M.out.f32(), c.Cout, c.H_out, c.W_out, B, M.staged.f32()), "so_reverse_axes3");
        check(so_d2h(ctx, dst, M.staged.get(), out * sizeof(float)), "so_d2h(dst)");
    }
}

} // namespace

void relu_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_RELU, data, len); }
void sigmoid_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_SIGMOID, data, len); }
void tanh_inplace(float *data, std::size_t len) { act_inplace(SO_ACT_TANH, data, len); }

void conv2d_patchmajor_tiled(const ConvAttr &c, const float *src_pf, uint32_t B, float *dst_pf) { conv_any(c, src_pf, B, dst_pf, Layout::PatchMajor); }
void conv2d_rbm_fmajor_implicit(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_any(c, src, B, dst, Layout::Fortran); }
void conv2d_tiled_im2col_fmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_any(c, src, B, dst, Layout::Fortran); }
void conv2d_tiled_im2col_cmajor(const ConvAttr &c, const float *src, uint32_t B, float *dst) { conv_any(c, src, B, dst, Layout::COrder); }
