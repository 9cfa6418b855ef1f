// Thin C++ conveniences over the C ABI of the HIP backend (cavs_hip.h): error
// translation and owning buffers.  The host runtime touches the device only
// through these; it has no HIP dependency of its own.
#ifndef CAVS_HOST_DEVICE_H_
#define CAVS_HOST_DEVICE_H_

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>

#include "cavs_hip.h"

namespace cavs {

struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

inline void check(int rc) {
  if (rc != CAVS_OK) throw Error(rc, cavs_last_error());
}

[[noreturn]] inline void fail(int code, const std::string &msg) { throw Error(code, msg); }

// Counts the times any DeviceArray let go of its storage: whoever keeps device addresses beyond a
// call (a recorded graph of launches) compares the count it saw with the current one.
inline std::atomic<uint64_t> &device_array_epoch() {
  static std::atomic<uint64_t> epoch{0};
  return epoch;
}

// Device array that only ever grows; contents are not preserved across growth
// (the reference's TensorBuffer::Resize behaves the same, cavs/midend/tensor.cc:44-50).
template <typename T>
class DeviceArray {
 public:
  DeviceArray() = default;
  DeviceArray(const DeviceArray &) = delete;
  DeviceArray &operator=(const DeviceArray &) = delete;
  ~DeviceArray() {
    if (p_) device_array_epoch()++;
    cavs_free(p_);
  }
  // returns true when the storage was reallocated
  bool reserve(size_t n) {
    if (n <= cap_) return false;
    if (p_) device_array_epoch()++;
    check(cavs_free(p_));
    p_ = nullptr;
    cap_ = 0;
    void *q = nullptr;
    check(cavs_malloc(&q, n * sizeof(T)));
    p_ = static_cast<T *>(q);
    cap_ = n;
    return true;
  }
  T *get() const { return p_; }
  size_t capacity() const { return cap_; }
  T *at(size_t i) const { return p_ + i; }
  void swap(DeviceArray &o) {  // (no storage is let go of)
    std::swap(p_, o.p_);
    std::swap(cap_, o.cap_);
  }

 private:
  T *p_ = nullptr;
  size_t cap_ = 0;
};

template <typename T>
class PinnedArray {
 public:
  PinnedArray() = default;
  PinnedArray(const PinnedArray &) = delete;
  PinnedArray &operator=(const PinnedArray &) = delete;
  ~PinnedArray() { cavs_host_free(p_); }
  void reserve(size_t n) {
    if (n <= cap_) return;
    check(cavs_host_free(p_));
    p_ = nullptr;
    cap_ = 0;
    void *q = nullptr;
    check(cavs_host_alloc(&q, n * sizeof(T)));
    p_ = static_cast<T *>(q);
    cap_ = n;
  }
  T *get() const { return p_; }

 private:
  T *p_ = nullptr;
  size_t cap_ = 0;
};

}  // namespace cavs
#endif
