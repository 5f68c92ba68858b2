// Shared by the translation units of libbikv_pagecopy.so: error plumbing and the per-device
// status block. Not installed.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bikv {

// Records a printf-style message for bikv_last_error() on this thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t e, const char* what);

// The host-mapped status block of a device is cut into banks of ST_SLOTS words. Two are fixed, one per
// kind of caller; the rest are handed out one per host stager, so that a wait judges the launches of its
// own stager only: a flag left behind by somebody's unchecked asynchronous launch cannot fail it,
// bikv_check_status() from another thread cannot clear a flag it is about to read, and a page id
// rejected in one stager's launch is never reported (or cleared) by another stager's wait.
enum : int {
  ST_BANK_SHARED = 0,   // the asynchronous entry points; read and cleared by bikv_check_status()
  ST_BANK_RING = 1,     // copies issued by the ring producer
  ST_BANK_DYNAMIC = 2,  // first bank that acquire_bank() hands out (one per bikv_stager)
  ST_BANKS = 256        // 256 banks x 8 words x 4 bytes = 8 KiB of pinned memory per device
};

// Device-side pointer of bank `bank` of the status block of `device` (created on first use).
int device_status(int device, int bank, uint32_t** dev_ptr);
// A bank of its own for a new stager (cleared), or BIKV_ERANGE when all are taken; release_bank() returns it.
int acquire_bank(int device, int* bank_out);
void release_bank(int device, int bank);

// Synchronises `stream`, then converts raised status slots of `bank` into BIKV_EBOUNDS (and clears them).
int sync_and_check(int device, int bank, hipStream_t stream);
// The same without the synchronisation, for callers that have drained their streams themselves.
int check_bank(int device, int bank);

// The run copy behind bikv_copy_runs[_ragged], reporting into a chosen status bank.
int copy_runs_banked(int bank, const void* src, int64_t src_bytes, void* dst, int64_t dst_bytes,
                     const int64_t* src_off, const int64_t* dst_off, const int64_t* run_len,
                     int64_t n_runs, int64_t run_bytes, int64_t unit_bytes, void* stream);

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
