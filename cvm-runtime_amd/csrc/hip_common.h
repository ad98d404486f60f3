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
void kernel_timing_mark(const char* name, double work, double bytes, const char* desc, hipStream_t s, bool start);

struct KernelTimer {
  const char* name;
  hipStream_t s;
  bool on;
  // `work` = algorithmic operations (or bytes) of this launch; `bytes` = algorithmic HBM bytes where the
  // work is counted in operations; `desc` = what the launch is (layer shape, kernel configuration)
  KernelTimer(const char* n, double work, hipStream_t st, double bytes = 0, const char* desc = nullptr)
      : name(n), s(st), on(kernel_timing_enabled()) {
    if (on) kernel_timing_mark(name, work, bytes, desc, s, true);
  }
  ~KernelTimer() {
    if (on) kernel_timing_mark(name, 0, 0, nullptr, s, false);
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

// A requantisation chain prepared for the device.  Every stage the graph can
// put behind a producer -- relu, cvm_clip, clip, and each regime of
// cvm_right_shift -- has the form
//     v = (clamp(v, lo, hi) >> s1) + add) >> s2          (add wraps)
//   relu            : clamp to [0, INT32_MAX]
//   clip / cvm_clip : clamp to [lo, hi]
//   cvm_right_shift : regime "saturate"  clamp to the pre-shifted bounds, s1 = 0, add = 2^(b-1), s2 = b
//                     (the rounding shift is monotonic and maps the bounds to -max / max, so
//                      clamping first equals the reference's compare-then-shift)
//                     regime "p + b >= 32"  no clamp, s1 = b-1, add = 1, s2 = 1
//                     regime "b >= 31"      no clamp, s1 = 31
//                     regime "max == 0"     clamp to [0, 0]
// so the device code is branch-free.  Adjacent pure clamps are merged on the host.
struct DevStage {
  int32_t lo, hi;
  int32_t s1, add, s2;
  int32_t mul;   // applied after the clamp, before the shifts (1 unless the stage is a multiplication)
};
struct DevChain {
  int count;
  DevStage st[4];
};

__device__ __forceinline__ int32_t apply_stage(const DevStage& s, int32_t v) {
  v = v < s.lo ? s.lo : v;
  v = v > s.hi ? s.hi : v;
  if (s.mul != 1) v = wmul(v, s.mul);   // uniform across the launch
  return wadd(v >> s.s1, s.add) >> s.s2;
}

__device__ __forceinline__ int32_t apply_chain(const DevChain& c, int32_t v) {
  // count is uniform across the launch: scalar branches only
  if (c.count > 0) v = apply_stage(c.st[0], v);
  if (c.count > 1) v = apply_stage(c.st[1], v);
  if (c.count > 2) v = apply_stage(c.st[2], v);
  if (c.count > 3) v = apply_stage(c.st[3], v);
  return v;
}

inline bool stage_is_clamp(const DevStage& s) { return s.s1 == 0 && s.add == 0 && s.s2 == 0 && s.mul == 1; }

// host: what a stage without a multiplication does to a value that already lies inside its clamp
inline int64_t stage_shift_part(const DevStage& s, int64_t v) { return ((v >> s.s1) + s.add) >> s.s2; }

// host: folds a pure clamp [clo, chi] that FOLLOWS stage p into p's own clamp, when that is exact for every input.
// On p's clamped domain [lo, hi] the shift part f(v) = ((v >> s1) + add) >> s2 never wraps (checked) and is monotonic
// with steps of at most one, so it takes every value between f(lo) and f(hi): clamping f's result to [clo, chi] then
// equals clamping the input to [lo', hi'], lo' the smallest v with f(v) >= clo and hi' the largest with f(v) <= chi.
inline bool merge_clamp_behind(DevStage* p, int32_t clo, int32_t chi) {
  if (p->mul != 1 || clo > chi || p->lo > p->hi) return false;
  if (p->s1 == 0 && p->s2 == 0) return false;   // not a shift: nothing says its steps are at most one
  const int64_t lo = p->lo, hi = p->hi;
  const int64_t a = (lo >> p->s1) + p->add, b = (hi >> p->s1) + p->add;
  if (a < INT32_MIN || a > INT32_MAX || b < INT32_MIN || b > INT32_MAX) return false;   // the add could wrap
  const int64_t flo = stage_shift_part(*p, lo), fhi = stage_shift_part(*p, hi);
  if (fhi < clo || flo > chi) return false;     // the result would be a constant: leave the two stages as they are
  int64_t nlo = lo, nhi = hi;
  if (flo < clo) {   // smallest v in (lo, hi] with f(v) >= clo
    int64_t l = lo, h = hi;   // f(l) < clo <= f(h)
    while (h - l > 1) {
      const int64_t m = l + (h - l) / 2;
      if (stage_shift_part(*p, m) >= clo) h = m; else l = m;
    }
    nlo = h;
  }
  if (fhi > chi) {   // largest v in [lo, hi) with f(v) <= chi
    int64_t l = lo, h = hi;   // f(l) <= chi < f(h)
    while (h - l > 1) {
      const int64_t m = l + (h - l) / 2;
      if (stage_shift_part(*p, m) <= chi) l = m; else h = m;
    }
    nhi = l;
  }
  if (nlo > nhi) return false;
  p->lo = (int32_t)nlo;
  p->hi = (int32_t)nhi;
  return true;
}

// host: validates and converts the C-ABI chain; returns false on a bad stage
inline bool make_chain(const cvmhip_chain* in, DevChain* out) {
  out->count = 0;
  if (!in) return true;
  if (in->count < 0 || in->count > 4) return false;
  for (int i = 0; i < in->count; ++i) {
    const cvmhip_stage& s = in->stage[i];
    DevStage d = {INT32_MIN, INT32_MAX, 0, 0, 0, 1};
    if (s.kind == CVMHIP_STAGE_RELU) {
      d.lo = 0;
    } else if (s.kind == CVMHIP_STAGE_CLIP) {
      // max(min(v, hi), lo): with lo > hi the result is always lo
      d.lo = s.lo;
      d.hi = s.hi < s.lo ? s.lo : s.hi;
    } else if (s.kind == CVMHIP_STAGE_RSHIFT) {
      if (s.precision < 1 || s.precision > 32 || s.shift_bit < 1 || s.shift_bit > 32) return false;
      const RShift r = make_rshift(s.precision, s.shift_bit);
      if (r.mode == 0) { d.lo = d.hi = 0; }
      else if (r.mode == 1) { d.s1 = 31; }
      else {
        d.s1 = r.sh; d.add = 1; d.s2 = 1;
        if (r.mode == 3) {
          // after the clamp v + 2^(b-1) cannot overflow, and ((v >> (b-1)) + 1) >> 1 == (v + 2^(b-1)) >> b
          d.lo = r.x_min; d.hi = r.x_max;
          d.s1 = 0; d.add = (int32_t)1 << r.sh; d.s2 = r.sh + 1;
        }
      }
    } else if (s.kind == CVMHIP_STAGE_MUL) {
      d.mul = s.lo;   // wrapping int32 product, as broadcast_mul computes it (broadcast.cc:75-86)
    } else if (s.kind == CVMHIP_STAGE_CLAMP_SHIFT) {
      if (s.shift_bit < 0 || s.shift_bit > 31 || s.lo > s.hi) return false;
      d.lo = s.lo; d.hi = s.hi; d.s2 = s.shift_bit;
    } else {
      return false;
    }
    // a pure clamp behind a shift stage becomes part of that stage's own clamp where that is exact
    if (out->count > 0 && stage_is_clamp(d) && !stage_is_clamp(out->st[out->count - 1]) &&
        merge_clamp_behind(&out->st[out->count - 1], d.lo, d.hi))
      continue;
    // merge a pure clamp into a preceding pure clamp, or into the clamp of the stage that follows it
    if (out->count > 0 && stage_is_clamp(out->st[out->count - 1])) {
      DevStage& p = out->st[out->count - 1];
      // clamp(clamp(v, p.lo, p.hi), d.lo, d.hi)
      int32_t lo = p.lo > d.lo ? p.lo : d.lo, hi = p.hi < d.hi ? p.hi : d.hi;
      if (lo > hi) lo = hi = (p.hi < d.lo ? d.lo : d.hi);  // disjoint ranges: constant result
      d.lo = lo;
      d.hi = hi;
      p = d;
    } else {
      out->st[out->count++] = d;
    }
  }
  return true;
}

}  // namespace cvmhip
#endif
