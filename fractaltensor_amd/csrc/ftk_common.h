// Shared helpers for the gfx950 kernels behind include/ftk.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>
#include <type_traits>

#include "../../include/ftk.h"

namespace ftk {

// ---- error reporting ------------------------------------------------------
// One message buffer per host thread; entry points return a code and leave the
// text here.  Kernel launch failures are turned into FTK_ERR_LAUNCH.
char* last_error_buffer();
constexpr int kErrLen = 512;

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), kErrLen, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(FTK_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FTK_OK;
}

#define FTK_HIP(call)                                                        \
  do {                                                                       \
    hipError_t e_ = (call);                                                  \
    if (e_ != hipSuccess)                                                    \
      return ::ftk::fail(FTK_ERR_LAUNCH, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)

// Set-up that a call site owes every device once (a function attribute is kept with the device's copy of the code
// object, so a process that drives two devices has to set it on both).  The set-up is idempotent: two threads that
// both find the device unprepared both do it.
class DeviceOnce {
 public:
  // true while the current device has not been prepared by this call site; *bit then goes to done()
  bool pending(unsigned* bit) const {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 31) {
      *bit = 0;
      return true;
    }
    *bit = 1u << dev;
    return !(seen_.load(std::memory_order_acquire) & *bit);
  }
  void done(unsigned bit) { seen_.fetch_or(bit, std::memory_order_release); }

 private:
  std::atomic<unsigned> seen_{0};
};

// The largest dynamic LDS size a call site has set on its kernel, per device: for launchers whose LDS need grows
// with the shape.  Two threads that both find the stored size too small both set the attribute; the larger one wins.
class DeviceMax {
 public:
  // true when the current device has not been given at least `value` by this call site; *dev then goes to raise()
  bool below(int value, int* dev) const {
    *dev = -1;
    int d = 0;
    if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= kDevices) return true;
    *dev = d;
    return max_[d].load(std::memory_order_acquire) < value;
  }
  void raise(int dev, int value) {
    if (dev < 0) return;
    int cur = max_[dev].load(std::memory_order_relaxed);
    while (cur < value && !max_[dev].compare_exchange_weak(cur, value, std::memory_order_release)) {
    }
  }

 private:
  static constexpr int kDevices = 32;
  std::atomic<int> max_[kDevices] = {};
};

// Every workspace a stacked-LSTM entry point takes starts with this block; its first int is the status word
// that ftk_stacked_lstm_status() reads.
constexpr size_t kStatusBytes = 256;

// Device properties, queried once per device id.
struct DeviceProps {
  int cus = 0;
  int lds_optin = 0;
  int clock_khz = 0;
  int wave = 0;
  char arch[32] = {0};
};
int device_props(const DeviceProps** out);

// ---- vector types for MFMA operands ----------------------------------------
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// Compile-time loop: the body sees its index as a constant expression
// (std::integral_constant), so register arrays indexed by it are promoted to
// registers even when the body sits under a runtime condition.
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// ---- device math ------------------------------------------------------------
// exp through the hardware base-2 exponential (about 1 ulp), reciprocal through
// v_rcp_f32 (1 ulp).  sigmoid is accurate to a few 1e-7 relative everywhere.
__device__ __forceinline__ float fast_exp(float x) {
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}

__device__ __forceinline__ float sigmoid_f(float x) {
  return __builtin_amdgcn_rcpf(1.0f + fast_exp(-x));
}

// tanh(x) = 1 - 2/(1+e^{2x}) loses relative accuracy near 0 (the result is the
// difference of two numbers close to 1), so small arguments use the odd Taylor
// polynomial instead; the switch point keeps both branches below 2e-7 relative.
__device__ __forceinline__ float tanh_f(float x) {
  const float big = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + fast_exp(2.0f * x));
  const float x2 = x * x;
  const float small =
      x * (1.0f + x2 * (-0.33333333333f + x2 * (0.13333333333f + x2 * (-0.05396825397f + x2 * 0.02186948854f))));
  return fabsf(x) < 0.25f ? small : big;
}

}  // namespace ftk
