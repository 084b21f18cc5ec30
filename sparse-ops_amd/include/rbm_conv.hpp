// Row-block-merged (RBM) re-encoding of an ELLPACK matrix: source-compatible with the reference's
// include/rbm_conv.hpp:8-31 (same struct names, members and builder signature).
//
// The rows are taken in blocks of Ct_max.  For one block, `krel` lists in ascending order the
// columns in which at least one of its rows has a nonzero (the union columns); the pairs of union
// column u -- (row inside the block, weight), rows ascending -- are pairs[colptr[u] .. colptr[u+1]).
// A kernel that walks krel once applies each gathered operand to every row of the block that uses
// it, and still gives each row its products in ascending column order.
//
// Addition: SparseOnnxModel builds this plan for the convolutions the reference builds it for
// (Cout >= 32 and K >= 64, src/sparse_onnx.cpp:499-502) and, unlike the reference at HEAD, runs it:
// see sparseops::upload_rbm (device.hpp) and so_conv_plan_set_rbm (sparseops_hip.h).
#pragma once

#include <cstdint>
#include <vector>

#include "aligned_buffer.hpp"
#include "ellpack_encoder.hpp"

struct RBMColPair {
    uint16_t row;   // row inside the block, 0 .. Ct-1
    float w;        // weight
};

struct RBMBlock {
    uint32_t M0;                    // first row (output channel) of the block
    uint32_t Ct;                    // rows in the block (<= Ct_max)
    std::vector<uint32_t> krel;     // union columns, ascending (length U)
    std::vector<uint32_t> colptr;   // U + 1 offsets into pairs
    std::vector<RBMColPair> pairs;  // all union columns' pairs, one after the other
    std::vector<float> bias;        // Ct values, or empty when built without bias
};

struct RBMPlan {
    uint32_t M;        // rows of the matrix (Cout)
    uint32_t N;        // columns (Cin * kH * kW)
    uint32_t Ct_max;   // block height used by the builder
    std::vector<RBMBlock> blocks;
};

/// Build the plan from an ELLPACK matrix whose rows hold their columns in ascending order (what
/// convert_to_ellpack produces).  Reference: src/layers/rbm_conv.cpp:7-73.
RBMPlan build_rbm_from_ellpack(const Ellpack &E, const float *bias_or_null, uint32_t Ct_max = 8);
