// build_rbm_from_ellpack: the host-side builder of the row-block-merged format
// (reference: src/layers/rbm_conv.cpp:7-73; same result, different construction).
//
// The rows of a block already hold their columns in ascending order, so the union is a k-way
// merge: every row keeps a cursor; the smallest column under any cursor is the next union column
// and the rows whose cursor shows it contribute its pairs, in row order.  No sort is needed.
#include "rbm_conv.hpp"

#include <algorithm>
#include <stdexcept>

RBMPlan build_rbm_from_ellpack(const Ellpack &E, const float *bias_or_null, uint32_t Ct_max)
{
    if (Ct_max == 0 || Ct_max > 65535) throw std::runtime_error("build_rbm_from_ellpack: Ct_max must be in 1..65535");
    RBMPlan plan;
    plan.M = E.m;
    plan.N = E.n;
    plan.Ct_max = Ct_max;
    plan.blocks.reserve((std::size_t(E.m) + Ct_max - 1) / Ct_max);
    std::vector<uint32_t> cursor(Ct_max);
    for (uint32_t first = 0; first < E.m; first += Ct_max) {
        RBMBlock blk;
        blk.M0 = first;
        blk.Ct = std::min(Ct_max, E.m - first);
        std::size_t stored = 0;
        for (uint32_t r = 0; r < blk.Ct; ++r) {
            cursor[r] = 0;
            stored += E.nnz[first + r];
        }
        blk.colptr.push_back(0);
        blk.pairs.reserve(stored);
        for (std::size_t done = 0; done < stored;) {
            uint32_t next = 0xffffffffu;                        // smallest column not yet merged
            for (uint32_t r = 0; r < blk.Ct; ++r)
                if (cursor[r] < E.nnz[first + r]) next = std::min(next, E.idx[std::size_t(first + r) * E.r + cursor[r]]);
            blk.krel.push_back(next);
            for (uint32_t r = 0; r < blk.Ct; ++r) {
                const std::size_t slot = std::size_t(first + r) * E.r + cursor[r];
                if (cursor[r] < E.nnz[first + r] && E.idx[slot] == next) {
                    blk.pairs.push_back(RBMColPair{uint16_t(r), E.Wd.ptr[slot]});
                    ++cursor[r];
                    ++done;
                }
            }
            blk.colptr.push_back(uint32_t(blk.pairs.size()));
        }
        if (bias_or_null) blk.bias.assign(bias_or_null + first, bias_or_null + first + blk.Ct);
        plan.blocks.push_back(std::move(blk));
    }
    return plan;
}
