// Host ELLPACK encoder/decoder.  Output is bit-identical to the reference's
// (src/ellpack_encoder.cpp:6-60): r = largest per-row count of entries that
// compare != 0.0f (so -0.0f is dropped and NaN is kept), values and column
// indices packed in ascending column order, unused slots hold 0.0f / 0.
#include "ellpack_encoder.hpp"

#include <algorithm>
#include <cstring>

Ellpack convert_to_ellpack(const float *W, uint32_t m, uint32_t n)
{
    std::vector<uint32_t> counts(m, 0u);
    uint32_t widest = 0;
    for (uint32_t i = 0; i < m; ++i) {
        const float *row = W + std::size_t(i) * n;
        uint32_t c = 0;
        for (uint32_t j = 0; j < n; ++j) c += (row[j] != 0.0f) ? 1u : 0u;
        counts[i] = c;
        widest = std::max(widest, c);
    }

    Ellpack E(m, n, widest);
    const std::size_t slots = std::size_t(m) * widest;
    if (slots) {
        std::memset(E.Wd.ptr, 0, slots * sizeof(float));
        std::memset(E.idx.data(), 0, slots * sizeof(uint32_t));
    }
    for (uint32_t i = 0; i < m; ++i) {
        const float *row = W + std::size_t(i) * n;
        float *wdst = E.Wd.ptr + std::size_t(i) * widest;
        uint32_t *idst = E.idx.data() + std::size_t(i) * widest;
        for (uint32_t j = 0; j < n; ++j) {
            const float v = row[j];
            if (v != 0.0f) {
                *wdst++ = v;
                *idst++ = j;
            }
        }
    }
    E.nnz = std::move(counts);
    return E;
}

void decode_from_ellpack(const Ellpack &E, float *W_out)
{
    const std::size_t total = std::size_t(E.m) * E.n;
    if (total) std::memset(W_out, 0, total * sizeof(float));
    for (uint32_t i = 0; i < E.m; ++i) {
        const float *w = E.Wd.ptr + std::size_t(i) * E.r;
        const uint32_t *c = E.idx.data() + std::size_t(i) * E.r;
        float *dst = W_out + std::size_t(i) * E.n;
        for (uint32_t k = 0, cnt = E.nnz[i]; k < cnt; ++k) dst[c[k]] = w[k];
    }
}
