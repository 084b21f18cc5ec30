// Host ELLPACK encoder/decoder.  Output is bit-identical to the reference's
// (src/ellpack_encoder.cpp:6-60): r = largest per-row count of entries that
// compare != 0.0f (so -0.0f is dropped and NaN is kept), values and column
// indices packed in ascending column order, unused slots hold 0.0f / 0.
// Rows are independent, so both passes are split over the host's cores
// (the reference scans the matrix twice on one thread).
#include "ellpack_encoder.hpp"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <thread>

namespace {

// Calls work(first_row, last_row) on disjoint row ranges covering [0, rows), on up to
// hardware_concurrency() threads when there are enough elements to pay for starting them.
template <typename Work>
void over_row_ranges(uint32_t rows, std::size_t elements, Work work)
{
    const unsigned hw = std::max(1u, std::thread::hardware_concurrency());
    const unsigned want = (unsigned)std::min<std::size_t>({(std::size_t)hw, (std::size_t)rows, elements >> 20});
    if (want <= 1) {
        work(0u, rows);
        return;
    }
    std::vector<std::thread> team;
    team.reserve(want - 1);
    const uint32_t per = (rows + want - 1) / want;
    for (unsigned t = 1; t < want; ++t) {
        const uint32_t lo = std::min(rows, t * per), hi = std::min(rows, lo + per);
        if (lo < hi) team.emplace_back([=] { work(lo, hi); });
    }
    work(0u, std::min(rows, per));
    for (auto &th : team) th.join();
}

} // namespace

Ellpack convert_to_ellpack(const float *W, uint32_t m, uint32_t n)
{
    const std::size_t cells = std::size_t(m) * n;

    // stored entries per row, and the widest row
    std::vector<uint32_t> stored(m, 0u);
    std::atomic<uint32_t> widest{0};
    over_row_ranges(m, cells, [&](uint32_t lo, uint32_t hi) {
        uint32_t local = 0;
        for (uint32_t i = lo; i < hi; ++i) {
            const float *src = W + std::size_t(i) * n;
            const uint32_t c = (uint32_t)std::count_if(src, src + n, [](float v) { return v != 0.0f; });
            stored[i] = c;
            local = std::max(local, c);
        }
        uint32_t seen = widest.load(std::memory_order_relaxed);
        while (local > seen && !widest.compare_exchange_weak(seen, local, std::memory_order_relaxed)) {}
    });

    const uint32_t r = widest.load();
    Ellpack E(m, n, r);
    float *vals = E.Wd.ptr;
    uint32_t *cols = E.idx.data();
    over_row_ranges(m, cells, [&](uint32_t lo, uint32_t hi) {
        for (uint32_t i = lo; i < hi; ++i) {
            const float *src = W + std::size_t(i) * n;
            const std::size_t base = std::size_t(i) * r;
            uint32_t k = 0;
            for (uint32_t j = 0; j < n && k < stored[i]; ++j)
                if (src[j] != 0.0f) {
                    vals[base + k] = src[j];
                    cols[base + k] = j;
                    ++k;
                }
            std::fill(vals + base + k, vals + base + r, 0.0f);      // padding: value 0, column 0
            std::fill(cols + base + k, cols + base + r, 0u);
        }
    });
    E.nnz.swap(stored);
    return E;
}

void decode_from_ellpack(const Ellpack &E, float *W_out)
{
    over_row_ranges(E.m, std::size_t(E.m) * E.n, [&](uint32_t lo, uint32_t hi) {
        for (uint32_t i = lo; i < hi; ++i) {
            float *dst = W_out + std::size_t(i) * E.n;
            std::fill(dst, dst + E.n, 0.0f);
            const std::size_t base = std::size_t(i) * E.r;
            for (uint32_t k = 0; k < E.nnz[i]; ++k) dst[E.idx[base + k]] = E.Wd.ptr[base + k];
        }
    });
}
