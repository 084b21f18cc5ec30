// ELLPACK container and host encoder: source-compatible with the reference's
// include/ellpack_encoder.hpp:6-32 (a caller may construct an Ellpack, read and write its
// members, and call the two free functions exactly as there).
//
// Layout: row i owns slots [i*r, (i+1)*r) of Wd and idx; its first nnz[i] slots hold the row's
// nonzero values and their column numbers in ascending column order, the rest hold 0.0f / 0.
// r is the largest nnz[i].  Xt (the reference's gather scratch for matvec) is allocated so that
// code touching it still works, and never read by this library.
//
// Addition: `device`, the matrix's copy in GPU memory.  ellpack_matmul / ellpack_matvec create it
// on first use from the members as they are at that moment; copies of the struct made afterwards
// share it.  The copy is not compared with the host arrays again: after writing to Wd, idx, nnz
// (or m, n, r) of an Ellpack that has already been used, call invalidate_device(), and the next
// kernel call uploads the members afresh.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <vector>

#include "aligned_buffer.hpp"

namespace sparseops { struct EllpackMirror; }

struct Ellpack {
    uint32_t m;                  // rows
    uint32_t n;                  // columns of the dense matrix
    uint32_t r;                  // slots per row
    AlignedBuffer Wd;            // m*r values
    std::vector<uint32_t> idx;   // m*r column numbers
    AlignedBuffer Xt;            // m*r floats, unused (see above)
    std::vector<uint32_t> nnz;   // m counts of stored nonzeros
    mutable std::shared_ptr<sparseops::EllpackMirror> device;

    Ellpack(uint32_t rows, uint32_t cols, uint32_t slots_per_row)
        : m(rows), n(cols), r(slots_per_row), Wd(slot_count(rows, slots_per_row)),
          idx(slot_count(rows, slots_per_row), 0u), Xt(slot_count(rows, slots_per_row)), nnz(rows, 0u)
    {
    }

    std::size_t slots() const { return slot_count(m, r); }
    /// Forget the GPU copy (this struct's reference to it): the next kernel call uploads again.
    void invalidate_device() const { device.reset(); }

  private:
    static std::size_t slot_count(uint32_t rows, uint32_t per_row) { return std::size_t(rows) * per_row; }
};

// Dense row-major m x n -> ELLPACK (reference: src/ellpack_encoder.cpp:6-44).
Ellpack convert_to_ellpack(const float *W, uint32_t m, uint32_t n);

// ELLPACK -> dense row-major m x n; W_out has room for m*n floats and is overwritten entirely
// (reference: src/ellpack_encoder.cpp:46-60).
void decode_from_ellpack(const Ellpack &E, float *W_out);
