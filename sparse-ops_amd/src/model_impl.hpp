// Private state of SparseOnnxModel, shared by the loader (sparse_onnx.cpp) and the
// executor (model_run.cpp).
#pragma once

#include <string>
#include <unordered_map>
#include <vector>

#include "device.hpp"
#include "ellpack_encoder.hpp"
#include "sparse_onnx.hpp"
#include "sparseops_hip.h"

namespace sparseops {

enum class Op { MatMul, Conv, Act, Add, MaxPool, GlobalAveragePool };

struct LayerPlan {
    Op op = Op::Act;
    std::string name;           // ONNX op_type, for describe()
    int in0 = -1, in1 = -1;     // arena slot ids of the inputs
    int out = -1;               // arena slot id of the output
    std::size_t out_features = 0;
    std::string out_tensor;     // tensor name produced (after fusion: the activation's output)

    // MatMul / Conv
    Ellpack *E = nullptr;       // owned by Impl::weights
    const so_ellpack *dE = nullptr;
    so_conv_plan *conv = nullptr;
    so_rbm *rbm = nullptr;      // Conv: the row-block-merged plan attached to `conv`, when one was built
    so_conv_geom cg{};
    std::vector<float> bias;    // host copy; device copy lives in Impl::bias_pool
    std::size_t bias_offset = 0;
    bool has_bias = false;
    int act = SO_ACT_NONE;      // fused epilogue, or the activation of an Act layer
    bool residual = false;      // Conv: in1 is added to the convolution before the activation

    // pools
    so_pool_geom pg{};
    std::size_t in_features = 0;
};

struct Slot {
    std::size_t features = 0;   // largest per-sample size of any tensor placed here
    std::size_t offset = 0;     // float offset into the arena for the current batch
};

} // namespace sparseops

struct SparseOnnxModel::Impl {
    std::vector<sparseops::LayerPlan> layers;
    std::vector<std::unique_ptr<Ellpack>> weights;
    std::vector<sparseops::Slot> slots;
    std::unordered_map<std::string, std::vector<int>> shape_map;  // per tensor, batch first
    std::string input_name, output_name;
    std::vector<int> input_dims;   // as declared by the graph, batch first
    std::vector<int> output_dims;  // shape of the graph output, batch first
    int input_slot = -1, output_slot = -1;
    std::size_t in_features = 0, out_features = 0;
    uint32_t batch = 0;            // samples per call, as the caller sees it
    uint32_t pbatch = 0;           // samples per row of every arena tensor: batch rounded up to 4, 8 or a multiple of 16
                                   // when the model has convolutions (their LDS-windowed kernel works on such batch tiles)
    bool has_conv = false;

    sparseops::DeviceBuffer bias_pool;   // all biases, contiguous
    sparseops::DeviceBuffer arena;       // all activation slots
    sparseops::DeviceBuffer stage_in, stage_out;  // staging for the caller's layouts (batch-major, or unpadded rows)
    sparseops::DeviceBuffer stage_mid;            // [features x batch] between a transpose and the padded arena rows
    so_graph *graph = nullptr;           // recorded layer chain (arena -> arena)
    bool use_graph = true;

    ~Impl();
    float *slot_ptr(int s) const { return arena.f32() + slots[s].offset; }
    void enqueue_layers() const;                             // one launch per layer, arena slot to arena slot
    void launch_chain() const;                               // graph replay or eager
    bool padded() const { return pbatch != batch; }
    void rows_in(const float *d_rows) const;                 // [in_features x batch] -> the input slot (rows padded with zeros)
    void rows_out(float *d_rows) const;                      // the output slot -> [out_features x batch]
};
