// Host-side helpers shared by the translation units that implement the C entry points.
#pragma once

#include "rg_internal.h"

namespace rg {

// Stores the message rg_last_error() returns on the calling thread.
void set_error(const char* fmt, ...);

static inline int hip_fail(hipError_t e, const char* what) {
  set_error("%s: %s", what, hipGetErrorString(e));
  return RG_EHIP;
}

#define RG_HIP(call)                                  \
  do {                                                \
    hipError_t e_ = (call);                           \
    if (e_ != hipSuccess) return hip_fail(e_, #call); \
  } while (0)

static inline int elem_size(int dtype) {
  switch (dtype) {
    case RG_F32: return 4;
    case RG_F16: return 2;
    case RG_BF16: return 2;
    default: return -1;
  }
}

static inline int64_t round_up(int64_t x, int64_t q) { return (x + q - 1) / q * q; }

// Makes the plan's device current for the scope of a call and restores the caller's.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) : prev_(-1), changed_(false) {
    if (hipGetDevice(&prev_) == hipSuccess && prev_ != device) changed_ = (hipSetDevice(device) == hipSuccess);
  }
  ~DeviceGuard() {
    if (changed_) (void)hipSetDevice(prev_);
  }

 private:
  int prev_;
  bool changed_;
};

static inline int check_pointer(const void* p, int esz, const char* which, int i) {
  if (p != nullptr && (reinterpret_cast<uintptr_t>(p) % (uintptr_t)esz) != 0) {
    set_error("%s[%d] = %p is not aligned to its %d-byte element", which, i, p, esz);
    return RG_EALIGN;
  }
  return RG_OK;
}

}  // namespace rg
