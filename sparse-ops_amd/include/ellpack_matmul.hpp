// Y = E * X + bias on the GPU, behind the reference's signatures
// (include/ellpack_matmul.hpp:14-43).  All pointers are HOST pointers owned by the
// caller: X is [n x C] row-major, bias has m entries or is nullptr, Y is [m x C]
// row-major.  Each call uploads X (and bias), runs the HIP kernel on the device
// copy of E (uploaded once, cached on the Ellpack) and downloads Y.
// Throws std::runtime_error when no HIP device is usable; there is no CPU path.
#pragma once

#include <cstdint>

#include "ellpack_encoder.hpp"

/// USE_MASK selected the masked AVX-512 tail path in the reference; the HIP kernel
/// predicates tail lanes itself, so the flag changes nothing.  FUSE_RELU fuses the
/// ReLU epilogue.
template <bool USE_MASK, bool FUSE_RELU>
void ellpack_matmul_fused(const Ellpack &E, const float *X, uint32_t C, const float *bias, float *Y);

extern template void ellpack_matmul_fused<false, false>(const Ellpack &, const float *, uint32_t, const float *, float *);
extern template void ellpack_matmul_fused<false, true>(const Ellpack &, const float *, uint32_t, const float *, float *);
extern template void ellpack_matmul_fused<true, false>(const Ellpack &, const float *, uint32_t, const float *, float *);
extern template void ellpack_matmul_fused<true, true>(const Ellpack &, const float *, uint32_t, const float *, float *);

inline void ellpack_matmul(const Ellpack &E, const float *X, uint32_t C, const float *bias, float *Y)
{
    ellpack_matmul_fused<true, false>(E, X, C, bias, Y);
}
