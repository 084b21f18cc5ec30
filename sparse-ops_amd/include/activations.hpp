// In-place activations over a host buffer, with the reference's signatures
// (include/activations.hpp:10-16; src/activations.cpp:20-68), executed on the GPU: the buffer is
// copied to HBM, so_act runs (max(x, 0); 1 / (1 + expf(-x)); tanhf(x)) and the result is copied
// back.  PCIe-bound convenience entry points: inside SparseOnnxModel the same math runs fused into
// the producing kernel's epilogue.  Throw std::runtime_error when no HIP device is usable.
#pragma once

#include <cstddef>

void relu_inplace(float *data, std::size_t len);
void sigmoid_inplace(float *data, std::size_t len);
void tanh_inplace(float *data, std::size_t len);
