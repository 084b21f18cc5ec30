// 64-byte aligned, move-only float buffer.  Same surface as the reference's
// AlignedBuffer (include/aligned_buffer.hpp:8-30: members `ptr` and `size`,
// throws std::bad_alloc); the allocation is left uninitialised.
#pragma once

#include <cstddef>
#include <cstdlib>
#include <new>
#include <utility>

struct AlignedBuffer {
    float *ptr = nullptr;
    std::size_t size = 0;

    AlignedBuffer() = default;
    explicit AlignedBuffer(std::size_t count) : size(count)
    {
        const std::size_t bytes = ((count * sizeof(float) + 63) / 64) * 64;
        ptr = static_cast<float *>(std::aligned_alloc(64, bytes ? bytes : 64));
        if (!ptr) throw std::bad_alloc();
    }
    ~AlignedBuffer() { std::free(ptr); }

    AlignedBuffer(const AlignedBuffer &) = delete;
    AlignedBuffer &operator=(const AlignedBuffer &) = delete;
    AlignedBuffer(AlignedBuffer &&other) noexcept
        : ptr(std::exchange(other.ptr, nullptr)), size(std::exchange(other.size, 0)) {}
    AlignedBuffer &operator=(AlignedBuffer &&other) noexcept
    {
        std::swap(ptr, other.ptr);
        std::swap(size, other.size);
        return *this;
    }
};
