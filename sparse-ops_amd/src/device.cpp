// Process-wide device context, RAII buffers and the Ellpack device mirror.
#include "device.hpp"

#include <new>

#include "ellpack_encoder.hpp"

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

} // namespace sparseops
