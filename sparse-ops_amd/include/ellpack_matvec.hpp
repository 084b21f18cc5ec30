// y = E * x + bias on the GPU, behind the reference's signature
// (include/ellpack_matvec.hpp:12-17).  Host pointers: x has n entries, bias has m
// entries or is nullptr, y has m entries.  Unlike the reference this call does not
// write E.Xt and is safe to call concurrently on one Ellpack from several
// threads of one process (calls are serialised on the device stream).
#pragma once

#include "ellpack_encoder.hpp"

void ellpack_matvec(const Ellpack &E, const float *x, const float *bias, float *y);
