// Device buffer with value semantics — the role culib::CUDA_ptr<T> plays in the
// reference (lib/CUDA_ptr.hpp:10-69), over et_malloc/et_free of the C ABI:
//   DeviceBuffer(n)            n zero-filled elements
//   DeviceBuffer(ptr, n)       copy of n elements from a host or a device pointer
//   DeviceBuffer(vector)       copy of a host vector
//   DeviceBuffer(n, value)     n elements set to value
//   copy = deep device-to-device copy, move = steal; get/size/dump/clear/set.
// As in the reference (cudaMemcpyDefault, lib/CUDA_ptr.hpp:18-31) the pointer
// constructor takes host or device memory: the runtime tells them apart by the address.
#pragma once
#include <cstddef>
#include <type_traits>
#include <vector>

#include "half.h"
#include "status.h"

namespace et {

template <typename T> class DeviceBuffer {
    static_assert(std::is_trivially_copyable<T>::value, "device buffers hold plain data");

  public:
    std::size_t size = 0;

    DeviceBuffer() = delete;
    explicit DeviceBuffer(std::size_t n) : size(n) { etChk(et_malloc(&raw_, bytes())); }
    DeviceBuffer(const T *host_or_device, std::size_t n) : size(n) {
        etChk(et_malloc(&raw_, bytes()));
        etChk(et_memcpy_auto(raw_, host_or_device, bytes()));
    }
    DeviceBuffer(const std::vector<T> &host) : DeviceBuffer(host.data(), host.size()) {}
    DeviceBuffer(std::size_t n, T value) : size(n) {
        etChk(et_malloc(&raw_, bytes()));
        set(value);
    }
    DeviceBuffer(const DeviceBuffer &other) : size(other.size) {
        etChk(et_malloc(&raw_, bytes()));
        etChk(et_memcpy_d2d(raw_, other.raw_, bytes(), nullptr));
        etChk(et_stream_sync(nullptr));
    }
    DeviceBuffer(DeviceBuffer &&other) noexcept : size(other.size), raw_(other.raw_) {
        other.raw_ = nullptr;
        other.size = 0;
    }
    DeviceBuffer &operator=(const DeviceBuffer &other) {
        if (this != &other) {
            DeviceBuffer tmp(other);
            swap(tmp);
        }
        return *this;
    }
    DeviceBuffer &operator=(DeviceBuffer &&other) noexcept {
        if (this != &other) {
            release();
            raw_ = other.raw_;
            size = other.size;
            other.raw_ = nullptr;
            other.size = 0;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    static DeviceBuffer from_device(const T *dev, std::size_t n) {
        DeviceBuffer b(n);
        etChk(et_memcpy_d2d(b.raw_, dev, b.bytes(), nullptr));
        etChk(et_stream_sync(nullptr));
        return b;
    }

    T *get() { return static_cast<T *>(raw_); }
    T *get() const { return static_cast<T *>(raw_); }
    std::size_t bytes() const { return size * sizeof(T); }

    void clear() {
        etChk(et_memset(raw_, 0, bytes(), nullptr));
        etChk(et_stream_sync(nullptr));
    }
    void dump(T *host) const {
        etChk(et_device_sync());
        etChk(et_memcpy_d2h(host, raw_, bytes()));
    }
    std::vector<T> to_host() const {
        std::vector<T> v(size);
        dump(v.data());
        return v;
    }
    void set(T value) {
        if constexpr (sizeof(T) == 2) {
            uint16_t bits;
            std::memcpy(&bits, &value, 2);
            etChk(et_fill_f16(reinterpret_cast<et_f16 *>(raw_), size, bits, nullptr));
        } else if constexpr (sizeof(T) == 4) {
            int32_t bits;
            std::memcpy(&bits, &value, 4);
            etChk(et_fill_i32(reinterpret_cast<int32_t *>(raw_), size, bits, nullptr));
        } else {
            std::vector<T> host(size, value);
            etChk(et_memcpy_h2d(raw_, host.data(), bytes()));
        }
        etChk(et_stream_sync(nullptr));
    }
    void swap(DeviceBuffer &other) noexcept {
        std::swap(raw_, other.raw_);
        std::swap(size, other.size);
    }

  private:
    void release() noexcept {
        if (raw_) (void)et_free(raw_);
        raw_ = nullptr;
    }
    void *raw_ = nullptr;
};

}  // namespace et

// The reference's spelling, so that callers written against it keep compiling.
namespace culib {
template <typename T> using CUDA_ptr = et::DeviceBuffer<T>;
}
