// Per-layer payloads with the reference's names and members (include/sparse_onnx.hpp:51-112), for
// callers that drive the layer kernels themselves (conv_kernels.hpp).  SparseOnnxModel keeps its own
// device-side plan and does not expose these.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "ellpack_encoder.hpp"
#include "rbm_conv.hpp"

namespace sparseops { struct ConvMirror; }

// What kind of node a layer is, and which operator exactly (include/sparse_onnx.hpp:30-47).
enum class LayerType { MatMul, Activation, Elementwise, Pool, Reshape, Conv };
enum class LayerOp { MatMul, Relu, Sigmoid, Tanh, Add, MaxPool, GlobalAveragePool, Flatten, Conv };
// Memory order of a 4-D activation (include/sparse_onnx.hpp:49): Fortran-order (B,C,H,W), C-order
// (B,C,H,W), or [C][H][W][B]; the conv2d_* entry points of conv_kernels.hpp take one each.
enum class DataLayout : uint8_t { BFastFortran, NCHW_C, PatchMajor };

struct MatMulAttr {
    Ellpack E;
    float *bias_ptr = nullptr;   // length E.m, or null
    bool fuse_relu = false;
};

struct KMap {
    uint32_t cin;
    int32_t dh;
    int32_t dw;
};

struct ConvAttr {
    Ellpack E;                   // Cout x K, K = Cin * kH * kW in (cin, kh, kw) order
    float *bias_ptr = nullptr;   // length Cout, or null

    uint32_t Cin = 0, Cout = 0, kH = 0, kW = 0;
    uint32_t stride_h = 1, stride_w = 1;
    uint32_t pad_h = 0, pad_w = 0;
    uint32_t dil_h = 1, dil_w = 1;
    uint32_t group = 1;
    uint32_t H_in = 0, W_in = 0;
    uint32_t H_out = 0, W_out = 0;

    // Kept for source compatibility; the GPU kernels derive every tap's address themselves and
    // read neither table (the reference fills them at load, src/sparse_onnx.cpp:440-497).
    std::vector<KMap> kmap;
    std::vector<std::size_t> patch_indices;
    std::size_t sentinel_off = 0;

    bool fuse_relu = false;
    RBMPlan rbm{};               // used when use_rbm is set and the plan is non-empty
    bool use_rbm{false};

    // Addition: what the conv2d_* entry points keep on the GPU for this layer between calls (the
    // convolution plan, the uploaded row-block-merged streams, staging buffers).  Built on the first
    // call and rebuilt when the geometry members, the batch, use_rbm or E's device copy change; after
    // editing `rbm` in place, call invalidate_device().
    mutable std::shared_ptr<sparseops::ConvMirror> device;
    void invalidate_device() const { device.reset(); }

    explicit ConvAttr(Ellpack e) : E(std::move(e)) {}
};

struct PoolAttr {
    int kH{1}, kW{1};
    int sH{1}, sW{1};
    int padH0{0}, padW0{0}, padH1{0}, padW1{0};
    bool is_global{false};
    uint32_t C{0}, H{0}, W{0};
    uint32_t H_out{0}, W_out{0};
};

struct FlattenAttr { int axis; };
struct AddAttr {};
struct ActAttr {};

// One node of a layer chain as a caller may assemble it (include/sparse_onnx.hpp:113-131): the
// payload for its kind plus the names of the graph values it reads and writes.
using LayerAttr = std::variant<MatMulAttr, ConvAttr, PoolAttr, FlattenAttr, AddAttr, ActAttr>;

struct Layer {
    LayerType type;
    LayerOp op;
    LayerAttr attr;
    std::vector<std::string> inputs;
    std::vector<std::string> outputs;
};

// A layer's result as the reference's per-layer helpers hand it on (include/sparse_onnx.hpp:134-138):
// `features` rows of the batch; `owned` says whether the receiver frees `data`.
struct RunResult {
    float *data;
    uint32_t features;
    bool owned;
};
