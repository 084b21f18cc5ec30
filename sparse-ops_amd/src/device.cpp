// Process-wide device context, RAII buffers and the Ellpack device mirror.
#include "device.hpp"

#include <new>
#include <vector>

#include "ellpack_encoder.hpp"
#include "rbm_conv.hpp"

namespace sparseops {

void check(so_status st, const char *what)
{
    if (st == SO_OK) return;
    if (st == SO_ERR_OOM) throw std::bad_alloc();
    throw std::runtime_error(std::string(what) + ": " + so_last_error());
}

namespace {
struct ContextHolder {
    so_ctx *ctx = nullptr;
    ~ContextHolder() { /* the context lives until process exit; HIP tears itself down */ }
};
ContextHolder g_holder;
std::mutex g_init_mutex;
std::mutex g_call_mutex;
} // namespace

so_ctx *context()
{
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (!g_holder.ctx) {
        so_ctx *ctx = nullptr;
        const so_status st = so_init(0, &ctx);
        if (st != SO_OK)
            throw std::runtime_error(std::string("sparseops: the HIP device path is unavailable and there is no "
                                                 "CPU fallback: ") + so_last_error());
        g_holder.ctx = ctx;
    }
    return g_holder.ctx;
}

std::mutex &context_mutex() { return g_call_mutex; }

DeviceBuffer::~DeviceBuffer() { release(); }

DeviceBuffer &DeviceBuffer::operator=(DeviceBuffer &&o) noexcept
{
    if (this != &o) {
        release();
        ptr_ = o.ptr_;
        bytes_ = o.bytes_;
        o.ptr_ = nullptr;
        o.bytes_ = 0;
    }
    return *this;
}

void DeviceBuffer::reserve(std::size_t bytes)
{
    if (ptr_ && bytes <= bytes_) return;
    release();
    void *p = nullptr;
    check(so_malloc(context(), bytes, &p), "so_malloc");
    ptr_ = p;
    bytes_ = bytes;
}

void DeviceBuffer::release()
{
    if (ptr_) {
        so_free(context(), ptr_);
        ptr_ = nullptr;
        bytes_ = 0;
    }
}

EllpackMirror::~EllpackMirror()
{
    if (handle) so_ellpack_free(context(), handle);
}

ConvMirror::~ConvMirror()
{
    if (plan) (void)so_conv_plan_free(context(), plan);
    if (rbm) (void)so_rbm_free(context(), rbm);
}

const so_ellpack *mirror(const Ellpack &E, int layouts)
{
    layouts |= SO_LAYOUT_ROW;
    if (E.device && (E.device->layouts & layouts) == layouts) return E.device->handle;
    if (E.device) layouts |= E.device->layouts;
    auto mir = std::make_shared<EllpackMirror>();
    check(so_ellpack_upload(context(), E.Wd.ptr, E.idx.data(), E.nnz.data(), E.m, E.n, E.r, layouts,
                            &mir->handle),
          "so_ellpack_upload");
    mir->layouts = layouts;
    E.device = std::move(mir);
    return E.device->handle;
}

so_rbm *upload_rbm(const RBMPlan &plan)
{
    std::vector<uint32_t> block_union{0}, krel, colptr{0};
    std::vector<uint16_t> pair_row;
    std::vector<float> pair_w;
    for (const RBMBlock &b : plan.blocks) {
        const uint32_t base = uint32_t(pair_w.size());
        krel.insert(krel.end(), b.krel.begin(), b.krel.end());
        for (std::size_t u = 1; u < b.colptr.size(); ++u) colptr.push_back(base + b.colptr[u]);
        for (const RBMColPair &q : b.pairs) {
            pair_row.push_back(q.row);
            pair_w.push_back(q.w);
        }
        block_union.push_back(uint32_t(krel.size()));
    }
    so_rbm *handle = nullptr;
    check(so_rbm_upload(context(), plan.M, plan.N, plan.Ct_max, uint32_t(plan.blocks.size()), block_union.data(), krel.data(),
                        colptr.data(), pair_row.data(), pair_w.data(), &handle),
          "so_rbm_upload");
    return handle;
}

} // namespace sparseops
