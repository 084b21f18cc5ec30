// The benchmark matrices' recipe, implemented once for the C++ harness (bench/bench_vendor.cpp) and
// for Python (sparseops_backend.benchmark_dense / benchmark_operand, python/datagen.py): the same
// seed gives the same matrix on both sides.  Recipe of the reference's drivers
// (benchmark-mkl/common/data_gen.cpp:23-96): each entry is kept with probability 1 - sparsity and
// then drawn from N(0, 1); with `irregular` the last row is fully dense; the dense operand is
// uniform in [-1, 1).  Random numbers come from std::mt19937_64 through explicit transforms (53-bit
// uniforms, Box-Muller normals): the standard library's distribution classes are not specified
// bit for bit across implementations, these are.
#pragma once

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <random>
#include <vector>

namespace sparseops_bench {

inline double uniform01(std::mt19937_64 &rng) { return double(rng() >> 11) * (1.0 / 9007199254740992.0); }   // [0, 1), 53 bits
inline float normal01(std::mt19937_64 &rng)
{
    const double u1 = 1.0 - uniform01(rng), u2 = uniform01(rng);                                              // u1 in (0, 1]
    return float(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925 * u2));
}

// Dense row-major M x N matrix with the given fraction of zeros.
inline std::vector<float> dense_matrix(int64_t M, int64_t N, double sparsity, uint64_t seed, bool irregular)
{
    std::vector<float> W(std::size_t(M) * std::size_t(N), 0.0f);
    std::mt19937_64 rng(seed);
    const double keep = 1.0 - sparsity;
    for (int64_t i = 0; i < M; ++i)
        for (int64_t j = 0; j < N; ++j)
            if ((irregular && i == M - 1) || uniform01(rng) < keep) W[std::size_t(i) * N + j] = normal01(rng);
    return W;
}

// The dense operand: `count` floats uniform in [-1, 1).
inline std::vector<float> dense_operand(std::size_t count, uint64_t seed)
{
    std::vector<float> X(count);
    std::mt19937_64 rng(seed);
    for (auto &v : X) v = float(2.0 * uniform01(rng) - 1.0);
    return X;
}

} // namespace sparseops_bench
