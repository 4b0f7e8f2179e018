// Device-memory plumbing for the host layer: checked HIP calls, an owning
// device buffer, host<->device copies and host-side bf16 conversion.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace vla {

struct HipError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw HipError(std::string(what) + ": " + hipGetErrorString(e));
}
#define VLA_HIP(expr) ::vla::hip_check((expr), #expr)

// Kernel-layer status (vla_kstatus) -> exception.
inline void k_check(int rc, const char* what) {
    if (rc != 0) throw std::runtime_error(std::string(what) + " returned vla_kstatus " + std::to_string(rc));
}
#define VLA_K(expr) ::vla::k_check((expr), #expr)

class DevBuf {
  public:
    DevBuf() = default;
    explicit DevBuf(size_t bytes) { alloc(bytes); }
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    DevBuf(DevBuf&& o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
    DevBuf& operator=(DevBuf&& o) noexcept {
        if (this != &o) { release(); p_ = o.p_; n_ = o.n_; o.p_ = nullptr; o.n_ = 0; }
        return *this;
    }
    ~DevBuf() { release(); }

    void alloc(size_t bytes) {
        release();
        if (bytes == 0) return;
        VLA_HIP(hipMalloc(&p_, bytes));
        n_ = bytes;
    }
    // Grow-only (contents are not preserved).
    void reserve(size_t bytes) { if (bytes > n_) alloc(bytes); }
    void zero() { if (p_) VLA_HIP(hipMemset(p_, 0, n_)); }
    void upload(const void* host, size_t bytes) {
        reserve(bytes);
        if (bytes) VLA_HIP(hipMemcpy(p_, host, bytes, hipMemcpyHostToDevice));
    }
    void download(void* host, size_t bytes) const {
        if (bytes) VLA_HIP(hipMemcpy(host, p_, bytes, hipMemcpyDeviceToHost));
    }
    void* get() const { return p_; }
    template <typename T> T* as() const { return static_cast<T*>(p_); }
    size_t bytes() const { return n_; }
    explicit operator bool() const { return p_ != nullptr; }

  private:
    void release() {
        if (p_) (void)hipFree(p_);
        p_ = nullptr;
        n_ = 0;
    }
    void* p_ = nullptr;
    size_t n_ = 0;
};

// Page-locked host staging memory (hipHostMalloc: allocated, never registered after the
// fact), grow-only.  Copies from it to the device are asynchronous to the host.
class PinnedBuf {
  public:
    PinnedBuf() = default;
    PinnedBuf(const PinnedBuf&) = delete;
    PinnedBuf& operator=(const PinnedBuf&) = delete;
    ~PinnedBuf() { release(); }
    void reserve(size_t bytes) {
        if (bytes <= n_) return;
        release();
        VLA_HIP(hipHostMalloc(&p_, bytes, hipHostMallocDefault));
        n_ = bytes;
    }
    void* get() const { return p_; }
    template <typename T> T* as() const { return static_cast<T*>(p_); }
    size_t bytes() const { return n_; }

  private:
    void release() {
        if (p_) (void)hipHostFree(p_);
        p_ = nullptr;
        n_ = 0;
    }
    void* p_ = nullptr;
    size_t n_ = 0;
};

// bf16 <-> f32 on the host, round to nearest even with NaN quieting.
inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline float bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// Uploads fp32 host data as `dtype` (0 = f32, 1 = bf16).
inline void upload_as(DevBuf& dst, const float* src, size_t n, int dtype) {
    if (dtype == 0) {
        dst.upload(src, n * sizeof(float));
    } else {
        std::vector<uint16_t> tmp(n);
        for (size_t i = 0; i < n; ++i) tmp[i] = f32_to_bf16(src[i]);
        dst.upload(tmp.data(), n * sizeof(uint16_t));
    }
}

inline size_t dtype_size(int dtype) { return dtype == 0 ? 4 : 2; }

// dst[i] = src[i] * scale in `dtype` (0 = f32, 1 = bf16, rounded as f32_to_bf16 does).  The
// bf16 form is written without a branch so that the compiler vectorises it.
inline void convert_scaled(void* dst, const float* src, size_t n, float scale, int dtype) {
    if (dtype == 0) {
        float* d = static_cast<float*>(dst);
        for (size_t i = 0; i < n; ++i) d[i] = src[i] * scale;
        return;
    }
    uint16_t* d = static_cast<uint16_t*>(dst);
    for (size_t i = 0; i < n; ++i) {
        const float f = src[i] * scale;
        uint32_t u;
        std::memcpy(&u, &f, 4);
        const uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
        const uint32_t quiet = (u >> 16) | 0x0040u;
        d[i] = (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u) ? quiet : rounded);
    }
}

}  // namespace vla
