// Minimal 2-D tensor with the shape of the reference's brotensor::Tensor as its attention call
// sites use it: {data, rows, cols, dtype, device}, row-major, caller-owned, resized in place by the
// ops, non-owning views (reference: src/dit/sana.cpp:90-93, include/brodiffusion/detail/device.h:21-25).
// Device memory comes from the C ABI (mi_malloc / mi_free); this header has no HIP in it.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "mi_attention.h"

namespace bdamd {

enum class Dtype { FP32, FP16, BF16, INT8 };
enum class Device { CPU, GPU };

inline std::size_t dtype_size(Dtype d) { return d == Dtype::FP32 ? 4 : (d == Dtype::INT8 ? 1 : 2); }

[[noreturn]] inline void fail(const std::string& msg) { throw std::runtime_error(msg); }

class Tensor {
public:
    void* data = nullptr;
    int rows = 0, cols = 0;
    Dtype dtype = Dtype::FP32;
    Device device = Device::GPU;

    Tensor() = default;
    Tensor(const Tensor&) = delete;             // views are made explicitly, never by accident
    Tensor& operator=(const Tensor&) = delete;
    Tensor(Tensor&& o) noexcept { *this = std::move(o); }
    Tensor& operator=(Tensor&& o) noexcept {
        if (this != &o) {
            release();
            data = o.data; rows = o.rows; cols = o.cols; dtype = o.dtype; device = o.device;
            owns_ = o.owns_; capacity_ = o.capacity_;
            o.data = nullptr; o.owns_ = false; o.capacity_ = 0; o.rows = o.cols = 0;
        }
        return *this;
    }
    ~Tensor() { release(); }

    std::size_t size() const { return static_cast<std::size_t>(rows) * cols; }
    std::size_t bytes() const { return size() * dtype_size(dtype); }

    // Non-owning view of rows [r0, r0 + n) or of caller memory.
    static Tensor view(Device dev, void* ptr, int r, int c, Dtype dt) {
        Tensor t; t.data = ptr; t.rows = r; t.cols = c; t.dtype = dt; t.device = dev; t.owns_ = false;
        return t;
    }
    Tensor row_view(int r0, int n) const {
        if (r0 < 0 || n < 0 || r0 + n > rows) fail("Tensor::row_view: rows out of range");
        return view(device, static_cast<char*>(data) + static_cast<std::size_t>(r0) * cols * dtype_size(dtype), n, cols, dtype);
    }

    // Keeps the allocation when it is large enough (no reallocation after warm-up).
    void resize(int r, int c, Dtype dt, Device dev = Device::GPU) {
        const std::size_t need = static_cast<std::size_t>(r) * c * dtype_size(dt);
        if (!owns_ && data != nullptr) {
            if (need > bytes() || dev != device) fail("Tensor::resize: cannot grow a view");
        } else if (need > capacity_ || dev != device) {
            release();
            if (dev == Device::GPU) {
                data = mi_malloc(need);
                if (!data) fail(std::string("Tensor::resize: ") + mi_last_error());
            } else {
                data = ::operator new(need ? need : 1);
            }
            owns_ = true; capacity_ = need;
        }
        rows = r; cols = c; dtype = dt; device = dev;
    }

    static Tensor from_host(const void* src, int r, int c, Dtype dt, Device dev = Device::GPU) {
        Tensor t; t.resize(r, c, dt, dev);
        if (dev == Device::GPU) {
            if (t.bytes() && mi_memcpy_h2d(t.data, src, t.bytes()) != 0) fail(std::string("Tensor::from_host: ") + mi_last_error());
        } else {
            std::char_traits<char>::copy(static_cast<char*>(t.data), static_cast<const char*>(src), t.bytes());
        }
        return t;
    }
    std::vector<std::uint8_t> to_host_bytes() const {
        std::vector<std::uint8_t> out(bytes());
        if (out.empty()) return out;
        if (device == Device::GPU) {
            if (mi_stream_synchronize(nullptr) != 0 || mi_memcpy_d2h(out.data(), data, out.size()) != 0)
                fail(std::string("Tensor::to_host_bytes: ") + mi_last_error());
        } else {
            std::char_traits<char>::copy(reinterpret_cast<char*>(out.data()), static_cast<const char*>(data), out.size());
        }
        return out;
    }

private:
    bool owns_ = false;
    std::size_t capacity_ = 0;
    void release() {
        if (owns_ && data) {
            if (device == Device::GPU) mi_free(data); else ::operator delete(data);
        }
        data = nullptr; owns_ = false; capacity_ = 0;
    }
};

}  // namespace bdamd
