// A C++ caller written against the reference's headers only (ellpack_encoder.hpp,
// ellpack_matmul.hpp, ellpack_matvec.hpp, activations.hpp, conv_kernels.hpp, rbm_conv.hpp, sparse_onnx.hpp): host pointers in, host pointers out,
// as benchmark-mkl/matmul/bench_matmul.cpp:98 and benchmark-mkl/matvec/bench_matvec.cpp:100 of the
// reference call them.  Checks every result against plain loops and exits non-zero on a mismatch.
//
//   dropin_consumer                      kernels only
//   dropin_consumer model.onnx in.bin expected.bin B     + SparseOnnxModel::run, bit for bit
#include "activations.hpp"
#include "conv_kernels.hpp"
#include "ellpack_encoder.hpp"
#include "ellpack_matmul.hpp"
#include "ellpack_matvec.hpp"
#include "rbm_conv.hpp"
#include "sparse_onnx.hpp"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <random>
#include <vector>

static int failures = 0;
static void check(bool ok, const char *what)
{
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    if (!ok) ++failures;
}

static std::vector<float> read_floats(const char *path)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    std::vector<float> v(f ? (size_t)f.tellg() / sizeof(float) : 0);
    f.seekg(0);
    f.read(reinterpret_cast<char *>(v.data()), (std::streamsize)(v.size() * sizeof(float)));
    return v;
}

int main(int argc, char **argv)
{
    const uint32_t m = 300, n = 200, C = 72;
    std::mt19937 rng(7);
    std::normal_distribution<float> gauss;
    std::uniform_real_distribution<float> coin(0.0f, 1.0f);
    std::vector<float> W(size_t(m) * n), X(size_t(n) * C), bias(m), x(n);
    for (auto &v : W) v = coin(rng) < 0.85f ? 0.0f : gauss(rng);
    for (auto &v : X) v = gauss(rng);
    for (auto &v : bias) v = gauss(rng);
    for (auto &v : x) v = gauss(rng);
    std::fill(W.begin() + 5 * n, W.begin() + 6 * n, 0.0f);          // an empty row

    Ellpack E = convert_to_ellpack(W.data(), m, n);
    std::vector<float> back(size_t(m) * n, -1.0f);
    decode_from_ellpack(E, back.data());
    check(std::memcmp(back.data(), W.data(), back.size() * sizeof(float)) == 0, "decode(encode(W)) == W");
    check(E.m == m && E.n == n && E.nnz[5] == 0 && E.Wd.size == size_t(m) * E.r && E.idx.size() == size_t(m) * E.r,
          "Ellpack members");

    // the reference's rounding sequence: bias, then one fused multiply-add per stored slot in order
    std::vector<float> want(size_t(m) * C), got(size_t(m) * C, NAN);
    for (uint32_t i = 0; i < m; ++i)
        for (uint32_t c = 0; c < C; ++c) {
            float acc = bias[i];
            for (uint32_t k = 0; k < E.nnz[i]; ++k) acc = std::fmaf(E.Wd.ptr[size_t(i) * E.r + k], X[size_t(E.idx[size_t(i) * E.r + k]) * C + c], acc);
            want[size_t(i) * C + c] = acc;
        }
    ellpack_matmul(E, X.data(), C, bias.data(), got.data());
    check(std::memcmp(got.data(), want.data(), got.size() * sizeof(float)) == 0, "ellpack_matmul bit-exact");

    std::fill(got.begin(), got.end(), NAN);
    ellpack_matmul_fused<false, true>(E, X.data(), C, bias.data(), got.data());
    bool relu_ok = true;
    for (size_t i = 0; i < got.size(); ++i) relu_ok &= got[i] == (want[i] > 0.0f ? want[i] : 0.0f);
    check(relu_ok, "ellpack_matmul_fused<false, true> (fused ReLU)");

    std::fill(got.begin(), got.end(), NAN);
    ellpack_matmul(E, X.data(), C, nullptr, got.data());
    bool nobias_ok = true;
    for (uint32_t i = 0; i < m && nobias_ok; ++i) {
        float acc = 0.0f;
        for (uint32_t k = 0; k < E.nnz[i]; ++k) acc = std::fmaf(E.Wd.ptr[size_t(i) * E.r + k], X[size_t(E.idx[size_t(i) * E.r + k]) * C], acc);
        nobias_ok = got[size_t(i) * C] == acc;
    }
    check(nobias_ok, "ellpack_matmul with bias == nullptr");

    std::vector<float> y(m, NAN);
    ellpack_matvec(E, x.data(), bias.data(), y.data());
    double worst = 0.0, scale = 0.0;
    for (uint32_t i = 0; i < m; ++i) {
        double acc = bias[i];
        for (uint32_t j = 0; j < n; ++j) acc += double(W[size_t(i) * n + j]) * x[j];
        worst = std::max(worst, std::fabs(acc - y[i]));
        scale = std::max(scale, std::fabs(acc));
    }
    check(worst <= 1e-5 * scale, "ellpack_matvec within 1e-5 of the fp64 product");

    // build_rbm_from_ellpack as the reference declares it (include/rbm_conv.hpp:31): every stored nonzero
    // appears once, under its column, in a block's union list; columns and rows ascend
    {
        const RBMPlan plan = build_rbm_from_ellpack(E, bias.data());
        std::vector<float> again(size_t(m) * n, 0.0f);
        bool ordered = plan.M == m && plan.N == n && plan.Ct_max == 8 && plan.blocks.size() == (m + 7) / 8;
        size_t pairs = 0;
        for (const RBMBlock &b : plan.blocks) {
            ordered &= b.colptr.size() == b.krel.size() + 1 && b.bias.size() == b.Ct && b.bias[0] == bias[b.M0];
            for (size_t u = 0; u < b.krel.size(); ++u) {
                ordered &= (u == 0 || b.krel[u] > b.krel[u - 1]) && b.colptr[u + 1] > b.colptr[u];
                for (uint32_t p = b.colptr[u]; p < b.colptr[u + 1]; ++p, ++pairs) {
                    ordered &= p == b.colptr[u] || b.pairs[p].row > b.pairs[p - 1].row;
                    again[size_t(b.M0 + b.pairs[p].row) * n + b.krel[u]] = b.pairs[p].w;
                }
            }
        }
        size_t stored = 0;
        for (uint32_t c : E.nnz) stored += c;
        check(ordered && pairs == stored && std::memcmp(again.data(), W.data(), again.size() * sizeof(float)) == 0,
              "build_rbm_from_ellpack: ordered, complete, decodes to W");
    }

    // activations.hpp (include/activations.hpp:10-16 of the reference): in place over a host buffer
    {
        std::vector<float> a(1000), r, sg, th;
        for (auto &v : a) v = 3.0f * gauss(rng);
        r = sg = th = a;
        relu_inplace(r.data(), r.size());
        sigmoid_inplace(sg.data(), sg.size());
        tanh_inplace(th.data(), th.size());
        bool ok = true;
        for (size_t i = 0; i < a.size(); ++i) {
            ok &= r[i] == (a[i] > 0.0f ? a[i] : 0.0f);
            ok &= std::fabs(sg[i] - 1.0f / (1.0f + std::exp(-a[i]))) <= 1e-6f;
            ok &= std::fabs(th[i] - std::tanh(a[i])) <= 1e-6f;
        }
        check(ok, "relu_inplace exact, sigmoid_inplace / tanh_inplace within 1e-6");
    }

    // conv_kernels.hpp (include/conv_kernels.hpp:8-36): the four entry points on their three layouts against
    // the direct definition (src/layers/conv.cpp:44-107: bias, then one fmaf per stored tap in slot order,
    // taps outside the image skipped)
    {
        const uint32_t Cin = 5, Cout = 40, kH = 3, kW = 3, H = 9, Wd_ = 11, B = 8, sh = 2, sw = 1, ph = 1, pw = 1;
        const uint32_t Ho = (H + 2 * ph - kH) / sh + 1, Wo = (Wd_ + 2 * pw - kW) / sw + 1, K = Cin * kH * kW;
        std::vector<float> Wc(size_t(Cout) * K), cb(Cout), src(size_t(Cin) * H * Wd_ * B);
        for (auto &v : Wc) v = coin(rng) < 0.6f ? 0.0f : gauss(rng);
        for (auto &v : cb) v = gauss(rng);
        for (auto &v : src) v = gauss(rng);
        ConvAttr c{convert_to_ellpack(Wc.data(), Cout, K)};
        c.bias_ptr = cb.data();
        c.Cin = Cin; c.Cout = Cout; c.kH = kH; c.kW = kW; c.stride_h = sh; c.stride_w = sw; c.pad_h = ph; c.pad_w = pw;
        c.H_in = H; c.W_in = Wd_; c.H_out = Ho; c.W_out = Wo;
        c.fuse_relu = true;
        std::vector<float> ref(size_t(Cout) * Ho * Wo * B);         // [C][H][W][B]
        for (uint32_t co = 0; co < Cout; ++co)
            for (uint32_t ho = 0; ho < Ho; ++ho)
                for (uint32_t wo = 0; wo < Wo; ++wo)
                    for (uint32_t b = 0; b < B; ++b) {
                        float acc = cb[co];
                        for (uint32_t s2 = 0; s2 < c.E.nnz[co]; ++s2) {
                            const uint32_t k = c.E.idx[size_t(co) * c.E.r + s2], ci = k / (kH * kW), kh = (k / kW) % kH, kw = k % kW;
                            const int hi = int(ho * sh + kh) - int(ph), wi = int(wo * sw + kw) - int(pw);
                            if (hi < 0 || wi < 0 || hi >= int(H) || wi >= int(Wd_)) continue;
                            acc = std::fmaf(c.E.Wd.ptr[size_t(co) * c.E.r + s2], src[((size_t(ci) * H + hi) * Wd_ + wi) * B + b], acc);
                        }
                        ref[((size_t(co) * Ho + ho) * Wo + wo) * B + b] = acc > 0.0f ? acc : 0.0f;
                    }
        std::vector<float> out(ref.size(), NAN);
        conv2d_patchmajor_tiled(c, src.data(), B, out.data());
        check(std::memcmp(out.data(), ref.data(), out.size() * sizeof(float)) == 0, "conv2d_patchmajor_tiled bit-exact");
        c.rbm = build_rbm_from_ellpack(c.E, cb.data());
        c.use_rbm = true;
        std::fill(out.begin(), out.end(), NAN);
        conv2d_patchmajor_tiled(c, src.data(), B, out.data());
        check(std::memcmp(out.data(), ref.data(), out.size() * sizeof(float)) == 0, "conv2d_patchmajor_tiled with the RBM plan attached");
        const void *state = c.device.get();      // plan, RBM streams and staging buffers, kept on the ConvAttr
        check(state != nullptr, "ConvAttr keeps its device state");
        // the same tensors in the Fortran (B,C,H,W) and the C-order (B,C,H,W) layouts
        std::vector<float> srcF(src.size()), srcC(src.size()), outF(ref.size(), NAN), outC(ref.size(), NAN);
        for (uint32_t ci = 0; ci < Cin; ++ci)
            for (uint32_t h = 0; h < H; ++h)
                for (uint32_t w = 0; w < Wd_; ++w)
                    for (uint32_t b = 0; b < B; ++b) {
                        const float v = src[((size_t(ci) * H + h) * Wd_ + w) * B + b];
                        srcF[b + size_t(B) * (ci + size_t(Cin) * (h + size_t(H) * w))] = v;
                        srcC[((size_t(b) * Cin + ci) * H + h) * Wd_ + w] = v;
                    }
        conv2d_rbm_fmajor_implicit(c, srcF.data(), B, outF.data());
        conv2d_tiled_im2col_cmajor(c, srcC.data(), B, outC.data());
        bool okF = true, okC = true;
        for (uint32_t co = 0; co < Cout; ++co)
            for (uint32_t h = 0; h < Ho; ++h)
                for (uint32_t w = 0; w < Wo; ++w)
                    for (uint32_t b = 0; b < B; ++b) {
                        const float v = ref[((size_t(co) * Ho + h) * Wo + w) * B + b];
                        okF &= outF[b + size_t(B) * (co + size_t(Cout) * (h + size_t(Ho) * w))] == v;
                        okC &= outC[((size_t(b) * Cout + co) * Ho + h) * Wo + w] == v;
                    }
        check(okF, "conv2d_rbm_fmajor_implicit (Fortran layout) bit-exact");
        std::fill(outF.begin(), outF.end(), NAN);
        conv2d_tiled_im2col_fmajor(c, srcF.data(), B, outF.data());
        bool okF2 = true;
        for (uint32_t co = 0; co < Cout; ++co)
            for (uint32_t h = 0; h < Ho; ++h)
                for (uint32_t w = 0; w < Wo; ++w)
                    for (uint32_t b = 0; b < B; ++b)
                        okF2 &= outF[b + size_t(B) * (co + size_t(Cout) * (h + size_t(Ho) * w))] == ref[((size_t(co) * Ho + h) * Wo + w) * B + b];
        check(okF2, "conv2d_tiled_im2col_fmajor bit-exact");
        check(okC, "conv2d_tiled_im2col_cmajor (C-order layout) bit-exact");
        check(c.device.get() == state, "repeated conv2d_* calls reuse the layer's device state");
    }

    {   // the reference's layer-chain types are declared with its names (include/sparse_onnx.hpp:30-138)
        PoolAttr pool;
        pool.kH = pool.kW = 3; pool.sH = pool.sW = 2; pool.C = 64;
        Layer L{LayerType::Pool, LayerOp::MaxPool, LayerAttr{pool}, {"x"}, {"y"}};
        RunResult rr{nullptr, 64u, false};
        const DataLayout lay = DataLayout::PatchMajor;
        check(std::get<PoolAttr>(L.attr).kH == 3 && L.inputs.size() == 1 && L.op == LayerOp::MaxPool && rr.features == 64u &&
              !rr.owned && lay != DataLayout::NCHW_C, "Layer / LayerAttr / RunResult / DataLayout");
    }

    if (argc == 5) {
        const uint32_t B = (uint32_t)std::atoi(argv[4]);
        const std::vector<float> in = read_floats(argv[2]), expected = read_floats(argv[3]);
        SparseOnnxModel model(argv[1]);
        const std::vector<size_t> shape = model.output_shape();
        size_t out_count = 1;
        for (size_t d : shape) out_count *= d;
        check(!shape.empty() && shape[0] == B && out_count == expected.size(), "SparseOnnxModel::output_shape");
        std::vector<float> out(expected.size(), NAN);
        model.run(in.data(), B, out.data());
        check(std::memcmp(out.data(), expected.data(), out.size() * sizeof(float)) == 0, "SparseOnnxModel::run bit-exact");
        model.resize_buffers(B);
        std::fill(out.begin(), out.end(), NAN);
        model.run(in.data(), B, out.data());
        check(std::memcmp(out.data(), expected.data(), out.size() * sizeof(float)) == 0, "run after resize_buffers");
    }
    std::printf("%d failure(s)\n", failures);
    return failures ? 1 : 0;
}
