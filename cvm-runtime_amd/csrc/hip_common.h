// Shared helpers for the HIP translation units (device code + launch checks).
#ifndef CVM_HIP_COMMON_H_
#define CVM_HIP_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/cvm_hip_ops.h"

#define CVM_MAXD 6

namespace cvmhip {

// Per-thread message for cvmhip_last_error().
void set_error(const char* fmt, ...);

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return CVMHIP_ERR_RUNTIME;
  }
  return CVMHIP_OK;
}

inline int arg_error(const char* what) {
  set_error("invalid argument: %s", what);
  return CVMHIP_ERR_ARG;
}

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Optional per-kernel timing (cvmhip_kernel_timing_begin/end): while enabled,
// launches bracketed by KernelTimer record a HIP event pair on the launch
// stream; totals per kernel name are read back when timing ends.
bool kernel_timing_enabled();
void kernel_timing_mark(const char* name, double work, hipStream_t s, bool start);

struct KernelTimer {
  const char* name;
  hipStream_t s;
  bool on;
  // `work` = algorithmic operations (or bytes) of this launch
  KernelTimer(const char* n, double work, hipStream_t st) : name(n), s(st), on(kernel_timing_enabled()) {
    if (on) kernel_timing_mark(name, work, s, true);
  }
  ~KernelTimer() {
    if (on) kernel_timing_mark(name, 0, s, false);
  }
};

// Grid for a grid-stride loop over `work` items with `block` threads: enough
// workgroups to put several waves on each of the 256 CUs, never more than needed.
inline unsigned grid_for(int64_t work, int block, int64_t cap = 256 * 16) {
  int64_t g = (work + block - 1) / block;
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return static_cast<unsigned>(g);
}

// int32 arithmetic that wraps modulo 2^32 (signed overflow is undefined in C++).
__device__ __forceinline__ int32_t wadd(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
__device__ __forceinline__ int32_t wsub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
__device__ __forceinline__ int32_t wmul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }

// Requantisation parameters prepared on the host once per launch.
// mode 0: max==0 -> 0;  1: b>=31 -> a>>31;  2: p+b>=32 -> rounding shift, no clip;
// 3: saturate on pre-shifted bounds, else rounding shift
// (src/runtime/cpu/ops/elemwise.cc:128-148).
struct RShift {
  int mode;
  int sh;  // shift_bit - 1
  int32_t lo, hi, x_min, x_max;
};

inline void prec_range(int precision, int32_t* lo, int32_t* hi) {
  int32_t mn = (int32_t)(-((((int64_t)1) << (precision - 1)) - 1));
  *lo = mn;
  *hi = (int32_t)(-(int64_t)mn);
}

inline RShift make_rshift(int precision, int shift_bit) {
  RShift r;
  prec_range(precision, &r.lo, &r.hi);
  r.sh = shift_bit - 1;
  r.x_min = r.x_max = 0;
  if (r.hi == 0) r.mode = 0;
  else if (shift_bit >= 31) r.mode = 1;
  else if (precision + shift_bit >= 32) r.mode = 2;
  else {
    r.mode = 3;
    r.x_min = (int32_t)((uint32_t)(-2 * r.hi - 1) << (shift_bit - 1));
    r.x_max = (int32_t)((uint32_t)(2 * r.hi - 1) << (shift_bit - 1));
  }
  return r;
}

__device__ __forceinline__ int32_t apply_rshift(const RShift& r, int32_t t) {
  switch (r.mode) {
    case 0: return 0;
    case 1: return t >> 31;
    case 2: return wadd(t >> r.sh, 1) >> 1;
    default:
      if (t < r.x_min) return r.lo;
      if (t > r.x_max) return r.hi;
      return ((t >> r.sh) + 1) >> 1;
  }
}

}  // namespace cvmhip
#endif
