// SparseOnnxModel: load an ONNX graph, ELLPACK-encode every FC / Conv weight,
// keep all layers resident in HBM and run inference as one chain of HIP kernels
// on one stream.  Public surface of the reference's class
// (include/sparse_onnx.hpp:139-163) plus resize_buffers, which the reference
// documents (README.md:146) but does not define.
//
// Activation layout (the reference's C++ contract, include/sparse_onnx.hpp:148-154):
// a tensor with per-sample shape S is stored as [prod(S) x B] row-major, batch
// contiguous; 4-D tensors are therefore [C][H][W][B].  Features are in C order of
// the per-sample shape, so Flatten is an alias and an FC layer after a 4-D Flatten
// needs no column permutation (the reference permutes for its (B,C,H,W)-Fortran
// layout, src/sparse_onnx.cpp:17-39).
//
// Supported ops (src/sparse_onnx.cpp:176-538): MatMul, Gemm, Conv (group 1), Relu,
// Sigmoid, Tanh, Add, MaxPool, GlobalAveragePool, Flatten (axis 1), Identity.
// Anything else throws std::runtime_error("Unsupported ONNX op: <op>").
// An activation that directly follows a MatMul/Gemm/Conv whose result has no other
// consumer is fused into that kernel's epilogue (the reference fuses Relu only,
// src/sparse_onnx.cpp:573-620; a fused Sigmoid/Tanh equals the separate layer).
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

class SparseOnnxModel {
public:
    /// Parse the model, encode and upload all weights, size the activation arena
    /// for the batch dimension of the graph input.  Throws std::runtime_error on
    /// parse errors, unsupported ops, dynamic shapes, or when no HIP device exists.
    explicit SparseOnnxModel(const std::string &onnx_path);
    ~SparseOnnxModel();
    SparseOnnxModel(SparseOnnxModel &&) noexcept;
    SparseOnnxModel &operator=(SparseOnnxModel &&) noexcept;

    /// input: host [input_features x B] row-major; output: host [output_features x B].
    /// B other than the current arena batch re-sizes the arena first (see
    /// resize_buffers); with an unchanged B the call allocates nothing.
    void run(const float *input, uint32_t B, float *output) const;

    /// Same, but input is batch-major (B, features...) C order -- what numpy and
    /// torch hold -- and output is (B, output features...) C order.  The two
    /// transposes run on the device.
    void run_batch_major(const float *input, uint32_t B, float *output) const;

    /// Device-pointer variant: dInput [input_features x B] and dOutput
    /// [output_features x B] are HBM pointers of the process-wide context; only
    /// kernels are enqueued, the call does not wait for them.
    void run_device(const float *dInput, uint32_t B, float *dOutput) const;

    /// (Re)allocate every activation buffer for `batch` samples and re-record the
    /// launch graph.  The only place that allocates after construction.
    void resize_buffers(uint32_t batch);

    /// Shape of the output tensor with the current batch first, e.g. {B, M}.
    std::vector<std::size_t> output_shape() const;
    std::vector<std::size_t> input_shape() const;
    uint32_t batch() const;
    std::size_t input_features() const;
    std::size_t output_features() const;

    /// Average milliseconds of one pass of the layer chain over the arena (input
    /// and output stay in HBM), measured with HIP events on the context's stream
    /// over `steps` back-to-back passes after `warmup` untimed ones.
    double time_device(int steps, int warmup) const;

    /// One line per executed layer, e.g. "MatMul 4096x784 r=109 act=relu bias=0".
    std::vector<std::string> describe() const;
    /// Sum over sparse layers of 2 * stored nonzeros * output columns per sample.
    double nnz_flops_per_sample() const;

    struct Impl;

private:
    std::unique_ptr<Impl> impl_;
};
