// C++ convenience layer over the C ABI (include/sparseops_hip.h): one process-wide
// context, RAII device buffers, and the translation of status codes into the
// exception types the reference's callers see (std::runtime_error).
#pragma once

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <stdexcept>
#include <string>

#include "sparseops_hip.h"

struct Ellpack;
struct RBMPlan;

namespace sparseops {

/// Throws std::runtime_error("<what>: <so_last_error()>") unless st == SO_OK
/// (std::bad_alloc for SO_ERR_OOM).
void check(so_status st, const char *what);

/// The process-wide context on device 0, created on first use.
/// Throws std::runtime_error if no HIP device is usable.
so_ctx *context();
/// Serialises host-pointer calls that share the staging buffers.
std::mutex &context_mutex();

class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(std::size_t bytes) { reserve(bytes); }
    ~DeviceBuffer();
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept;

    /// Grow-only: reallocates (contents lost) when `bytes` exceeds the capacity.
    void reserve(std::size_t bytes);
    void release();
    float *f32() const { return static_cast<float *>(ptr_); }
    void *get() const { return ptr_; }
    std::size_t bytes() const { return bytes_; }

private:
    void *ptr_ = nullptr;
    std::size_t bytes_ = 0;
};

/// Device copy of an Ellpack, owned through Ellpack::device.
struct EllpackMirror {
    so_ellpack *handle = nullptr;
    int layouts = 0;
    ~EllpackMirror();
};

/// What a ConvAttr keeps on the GPU between calls of the conv2d_* entry points (ConvAttr::device).
struct ConvMirror {
    so_conv_plan *plan = nullptr;
    so_rbm *rbm = nullptr;
    const void *ellpack = nullptr;        // the EllpackMirror the plan was built from
    uint32_t geom[14] = {0};              // so_conv_geom as built
    uint32_t tuned_batch = 0;
    bool with_rbm = false;
    DeviceBuffer in, out, bias, staged;   // grow-only: a repeated call allocates nothing
    ~ConvMirror();
};

/// Upload E once (or again if `layouts` asks for more than is resident) and
/// return the device handle.
const so_ellpack *mirror(const Ellpack &E, int layouts);

/// The row-block-merged plan handed to the device library (so_rbm_upload): its per-block vectors
/// laid end to end.  The caller owns the handle (so_rbm_free).  Biases stay with the caller: the
/// kernels take them per call.
so_rbm *upload_rbm(const RBMPlan &plan);

/// Device layouts to keep for Y = E * X with C dense columns: ROW, plus for large matrices and wide X
/// either TILED (bit-identical to the reference) or, with `fast`, RBM (row-block-merged: the fastest
/// kernel, results equal to fp32 round-off).
int matmul_layouts(const Ellpack &E, uint32_t C, bool fast);

} // namespace sparseops
