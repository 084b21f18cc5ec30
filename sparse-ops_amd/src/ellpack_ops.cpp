// Host-pointer entry points with the reference's signatures, executed on the GPU:
// device copy of E (cached) + upload of X/bias + HIP kernel + download of Y.
#include "ellpack_matmul.hpp"
#include "ellpack_matvec.hpp"

#include "device.hpp"

namespace {

// Grow-only staging buffers shared by all host-pointer calls of the process.
struct Staging {
    sparseops::DeviceBuffer x, y, bias;
};
Staging &staging()
{
    static Staging *s = new Staging();  // intentionally leaked: freed with the process
    return *s;
}

} // namespace

namespace sparseops {
// Device layouts worth keeping for Y = E * X with C dense columns.  Large, reasonably filled
// matrices and wide X pay for a second copy: the K-tiled one (LDS-staged kernel, the reference's
// bits) or, with `fast`, the row-block-merged one (the fastest kernel; sums in another order,
// accurate to fp32 round-off).
int matmul_layouts(const Ellpack &E, uint32_t C, bool fast)
{
    uint64_t total = 0;
    for (uint32_t c : E.nnz) total += c;
    const bool big = E.m >= 512 && E.n >= 512 && total >= 32ull * E.m;
    if (!big || C < 64) return SO_LAYOUT_ROW;
    // The row-block-merged kernel pays its fixed costs (sums over 12 or 24 streams) only with enough columns per
    // stream: below ~1500 columns the K-tiled kernel is ahead (4096 x 784 x 256: 11.2 us against 13.8).
    if (fast && E.n >= 1536) return SO_LAYOUT_ROW | SO_LAYOUT_RBM;
    return C % 4 == 0 ? (SO_LAYOUT_ROW | SO_LAYOUT_TILED) : SO_LAYOUT_ROW;
}
} // namespace sparseops

namespace {
using sparseops::matmul_layouts;

void matmul_host(const Ellpack &E, const float *X, uint32_t C, const float *bias, float *Y, int act)
{
    using namespace sparseops;
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (E.m == 0 || C == 0) return;
    const so_ellpack *dE = mirror(E, matmul_layouts(E, C, false));     // host-pointer calls are PCIe-bound: keep the reference's bits
    Staging &st = staging();
    const std::size_t xbytes = std::size_t(E.n) * C * sizeof(float);
    const std::size_t ybytes = std::size_t(E.m) * C * sizeof(float);
    st.x.reserve(xbytes);
    st.y.reserve(ybytes);
    check(so_h2d(ctx, st.x.get(), X, xbytes), "so_h2d(X)");
    const float *dBias = nullptr;
    if (bias) {
        st.bias.reserve(std::size_t(E.m) * sizeof(float));
        check(so_h2d(ctx, st.bias.get(), bias, std::size_t(E.m) * sizeof(float)), "so_h2d(bias)");
        dBias = st.bias.f32();
    }
    check(so_matmul(ctx, dE, st.x.f32(), C, dBias, st.y.f32(), act), "so_matmul");
    check(so_d2h(ctx, Y, st.y.get(), ybytes), "so_d2h(Y)");
}

} // namespace

template <bool USE_MASK, bool FUSE_RELU>
void ellpack_matmul_fused(const Ellpack &E, const float *X, uint32_t C, const float *bias, float *Y)
{
    matmul_host(E, X, C, bias, Y, FUSE_RELU ? SO_ACT_RELU : SO_ACT_NONE);
}

template void ellpack_matmul_fused<false, false>(const Ellpack &, const float *, uint32_t, const float *, float *);
template void ellpack_matmul_fused<false, true>(const Ellpack &, const float *, uint32_t, const float *, float *);
template void ellpack_matmul_fused<true, false>(const Ellpack &, const float *, uint32_t, const float *, float *);
template void ellpack_matmul_fused<true, true>(const Ellpack &, const float *, uint32_t, const float *, float *);

void ellpack_matvec(const Ellpack &E, const float *x, const float *bias, float *y)
{
    using namespace sparseops;
    so_ctx *ctx = context();
    std::lock_guard<std::mutex> lock(context_mutex());
    if (E.m == 0) return;
    // Skewed row lengths (widest row far above the mean): keep length classes so
    // that padding is never streamed and short rows do not occupy whole waves.
    uint64_t total = 0;
    for (uint32_t c : E.nnz) total += c;
    const bool skewed = uint64_t(E.r) * E.m > 2 * total + E.m;
    // Up to 65536 columns fit 16 bits: the device keeps them that way as well and the product streams
    // 6 bytes per nonzero instead of 8 (same bits).  On those the length-class kernel is the faster one for
    // even rows too while a wave gets only a few rows; so_matvec chooses between the two (layout 0).
    const int compact = E.n <= 65536u ? SO_LAYOUT_IDX16 : 0;
    const so_ellpack *dE = mirror(E, ((skewed || compact) ? (SO_LAYOUT_ROW | SO_LAYOUT_BINS) : SO_LAYOUT_ROW) | compact);
    Staging &st = staging();
    st.x.reserve(std::size_t(E.n) * sizeof(float));
    st.y.reserve(std::size_t(E.m) * sizeof(float));
    check(so_h2d(ctx, st.x.get(), x, std::size_t(E.n) * sizeof(float)), "so_h2d(x)");
    const float *dBias = nullptr;
    if (bias) {
        st.bias.reserve(std::size_t(E.m) * sizeof(float));
        check(so_h2d(ctx, st.bias.get(), bias, std::size_t(E.m) * sizeof(float)), "so_h2d(bias)");
        dBias = st.bias.f32();
    }
    check(so_matvec(ctx, dE, st.x.f32(), dBias, st.y.f32(), 0), "so_matvec");
    check(so_d2h(ctx, y, st.y.get(), std::size_t(E.m) * sizeof(float)), "so_d2h(y)");
}
