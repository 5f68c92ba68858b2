// Shared by the translation units of libbikv_pagecopy.so: error plumbing and the per-device
// status block. Not installed.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bikv {

// Records a printf-style message for bikv_last_error() on this thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t e, const char* what);

// Device-side pointer of the host-mapped status block of `device` (created on first use).
int device_status(int device, uint32_t** dev_ptr);

// Synchronises `stream`, then converts raised status slots into BIKV_EBOUNDS.
int sync_and_check(int device, hipStream_t stream);

// Makes `device` current for the scope and puts the caller's device back afterwards, so that an
// entry point never changes the current device of the thread that called it.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) {
    if (hipGetDevice(&prev_) != hipSuccess) prev_ = -1;
    if (prev_ != device) {
      err_ = hipSetDevice(device);
      changed_ = err_ == hipSuccess && prev_ >= 0;
    }
  }
  ~DeviceGuard() {
    if (changed_) (void)hipSetDevice(prev_);
  }
  DeviceGuard(const DeviceGuard&) = delete;
  DeviceGuard& operator=(const DeviceGuard&) = delete;
  hipError_t error() const { return err_; }

 private:
  int prev_ = -1;
  bool changed_ = false;
  hipError_t err_ = hipSuccess;
};

}  // namespace bikv

#define BIKV_DEVICE(device)                 \
  ::bikv::DeviceGuard bikv_guard_(device);  \
  BIKV_HIP(bikv_guard_.error())

#define BIKV_HIP(call)                                            \
  do {                                                            \
    hipError_t bikv_e_ = (call);                                  \
    if (bikv_e_ != hipSuccess) return ::bikv::fail_hip(bikv_e_, #call); \
  } while (0)
