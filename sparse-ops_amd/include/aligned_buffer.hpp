// Float storage on a 64-byte boundary with single ownership.  Source-compatible with the
// reference's AlignedBuffer (include/aligned_buffer.hpp:8-30): public `ptr` and `size`,
// construction from an element count, std::bad_alloc on failure, movable but not copyable.
// Contents start uninitialised.
#pragma once

#include <cstddef>
#include <cstdlib>
#include <new>

struct AlignedBuffer {
    static constexpr std::size_t kAlign = 64;

    float *ptr;
    std::size_t size;

    AlignedBuffer() noexcept : ptr(nullptr), size(0) {}

    explicit AlignedBuffer(std::size_t count) : ptr(nullptr), size(count)
    {
        // posix_memalign accepts any size, zero included (a distinct pointer that free() takes)
        void *mem = nullptr;
        if (posix_memalign(&mem, kAlign, count ? count * sizeof(float) : kAlign) != 0) throw std::bad_alloc();
        ptr = static_cast<float *>(mem);
    }

    AlignedBuffer(AlignedBuffer &&from) noexcept : AlignedBuffer() { take(from); }

    AlignedBuffer &operator=(AlignedBuffer &&from) noexcept
    {
        if (this != &from) {
            drop();
            take(from);
        }
        return *this;
    }

    AlignedBuffer(const AlignedBuffer &) = delete;
    AlignedBuffer &operator=(const AlignedBuffer &) = delete;

    ~AlignedBuffer() { drop(); }

  private:
    void drop() noexcept
    {
        std::free(ptr);
        ptr = nullptr;
        size = 0;
    }
    void take(AlignedBuffer &from) noexcept
    {
        ptr = from.ptr;
        size = from.size;
        from.ptr = nullptr;
        from.size = 0;
    }
};
