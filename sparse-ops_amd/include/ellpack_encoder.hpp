// ELLPACK container and host encoder.  Drop-in for the reference's
// include/ellpack_encoder.hpp:6-32: same struct members, same free functions.
// The one addition is `device`, an opaque handle to the matrix's copy in HBM,
// created on first use by ellpack_matmul / ellpack_matvec and shared by copies.
#pragma once

#include <cstdint>
#include <memory>
#include <vector>

#include "aligned_buffer.hpp"

namespace sparseops { struct EllpackMirror; }

struct Ellpack {
    uint32_t m;  ///< rows
    uint32_t n;  ///< columns of the dense matrix
    uint32_t r;  ///< slots per row = max nonzeros of any row

    AlignedBuffer Wd;           ///< m*r values, row-major, zero padded
    std::vector<uint32_t> idx;  ///< m*r column indices, zero padded
    AlignedBuffer Xt;           ///< m*r floats; host scratch kept for source compatibility, unused here
    std::vector<uint32_t> nnz;  ///< m stored-nonzero counts

    mutable std::shared_ptr<sparseops::EllpackMirror> device;  ///< HBM copy, lazily created

    Ellpack(uint32_t m_, uint32_t n_, uint32_t r_)
        : m(m_), n(n_), r(r_), Wd(std::size_t(m_) * r_), idx(std::size_t(m_) * r_),
          Xt(std::size_t(m_) * r_), nnz(m_) {}
};

/// Encode a dense row-major m x n matrix (reference: src/ellpack_encoder.cpp:6-44).
Ellpack convert_to_ellpack(const float *W, uint32_t m, uint32_t n);

/// Decode into a dense m x n matrix; W_out holds m*n floats
/// (reference: src/ellpack_encoder.cpp:46-60).
void decode_from_ellpack(const Ellpack &E, float *W_out);
