// Host-side plumbing of the C++ layer classes: error wrappers and an owning device array.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/linmt_hip.h"

namespace linmt {

// The reference's CudaErrorWrapper / CublasErrorWrapper / CudaGetLastError print the message and
// exit(EXIT_FAILURE) (src/utility_cu.cu:171-214).  Here the failure is raised as an exception with
// the same message: uncaught it terminates the process just the same, and the C facade used by the
// tests turns it into an error status instead of killing the test runner.
struct LinmtError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void HipErrorWrapper(hipError_t e, const char *msg) {
  if (e != hipSuccess) {
    std::string m = std::string("Error: ") + msg + ": " + hipGetErrorString(e);
    fprintf(stderr, "%s\n", m.c_str());
    throw LinmtError(m);
  }
}

inline void LhErrorWrapper(int status, const char *msg) {
  if (status != LH_OK) {
    std::string m = std::string("Error: ") + msg + " (status " + std::to_string(status) +
                    "): " + lh_last_error();
    fprintf(stderr, "%s\n", m.c_str());
    throw LinmtError(m);
  }
}

// Owning device buffer (the reference cudaMalloc's per object and never frees; this frees).
template <typename T>
class DeviceArray {
 public:
  DeviceArray() = default;
  explicit DeviceArray(size_t n) { Alloc(n); }
  DeviceArray(const DeviceArray &) = delete;
  DeviceArray &operator=(const DeviceArray &) = delete;
  DeviceArray(DeviceArray &&o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
  DeviceArray &operator=(DeviceArray &&o) noexcept {
    if (this != &o) {
      Free();
      p_ = o.p_; n_ = o.n_;
      o.p_ = nullptr; o.n_ = 0;
    }
    return *this;
  }
  ~DeviceArray() { Free(); }

  void Alloc(size_t n) {
    Free();
    n_ = n;
    if (n == 0) return;
    HipErrorWrapper(hipMalloc(reinterpret_cast<void **>(&p_), n * sizeof(T)),
                    "GPU memory allocation failed");
  }
  // Grow-only: keeps the buffer when it already holds n elements (contents are not kept otherwise).
  void Reserve(size_t n) {
    if (n > n_) Alloc(n);
  }
  void Free() {
    if (p_) (void)hipFree(p_);
    p_ = nullptr;
    n_ = 0;
  }
  void Zero(hipStream_t s) {
    if (n_) HipErrorWrapper(hipMemsetAsync(p_, 0, n_ * sizeof(T), s), "GPU memset failed");
  }
  void Zero(hipStream_t s, size_t n) {
    if (n > n_) throw LinmtError("DeviceArray::Zero out of range");
    if (n) HipErrorWrapper(hipMemsetAsync(p_, 0, n * sizeof(T), s), "GPU memset failed");
  }
  void Upload(const T *host, size_t n, hipStream_t s, size_t offset = 0) {
    if (n + offset > n_) throw LinmtError("DeviceArray::Upload out of range");
    if (n) HipErrorWrapper(hipMemcpyAsync(p_ + offset, host, n * sizeof(T), hipMemcpyHostToDevice, s),
                           "GPU memcpy H2D failed");
  }
  void Download(T *host, size_t n, hipStream_t s, size_t offset = 0) const {
    if (n + offset > n_) throw LinmtError("DeviceArray::Download out of range");
    if (n) HipErrorWrapper(hipMemcpyAsync(host, p_ + offset, n * sizeof(T), hipMemcpyDeviceToHost, s),
                           "GPU memcpy D2H failed");
  }
  T *get() const { return p_; }
  size_t size() const { return n_; }

 private:
  T *p_ = nullptr;
  size_t n_ = 0;
};

// Page-locked host buffer (allocated as such: registering existing memory is not available
// everywhere), grow-only: what asynchronous copies of a repeated call read and write.
template <typename T>
class PinnedArray {
 public:
  PinnedArray() = default;
  PinnedArray(const PinnedArray &) = delete;
  PinnedArray &operator=(const PinnedArray &) = delete;
  ~PinnedArray() {
    if (p_) (void)hipHostFree(p_);
  }
  void Reserve(size_t n) {
    if (n <= n_) return;
    if (p_) (void)hipHostFree(p_);
    p_ = nullptr;
    n_ = 0;
    HipErrorWrapper(hipHostMalloc(reinterpret_cast<void **>(&p_), n * sizeof(T), hipHostMallocDefault),
                    "page-locked host memory allocation failed");
    n_ = n;
  }
  T *get() const { return p_; }
  size_t size() const { return n_; }
  T &operator[](size_t i) const { return p_[i]; }

 private:
  T *p_ = nullptr;
  size_t n_ = 0;
};

}  // namespace linmt
