// Bandwidth-bound CVM operators for gfx950: elementwise, broadcast, pooling,
// reductions and index-remap copies.  Every kernel is a coalesced grid-stride
// sweep; int32 in, int32 out, bit-identical to the reference CPU operators.
#include <stdarg.h>

#include "hip_common.h"

namespace cvmhip {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---------------------------------------------------------------- unary ops
struct FRelu { __device__ int32_t operator()(int32_t v) const { return v < 0 ? 0 : v; } };
struct FClip {  // cvm_clip and clip: max(min(v, hi), lo)
  int32_t lo, hi;
  __device__ int32_t operator()(int32_t v) const { v = v < hi ? v : hi; return v > lo ? v : lo; }
};
struct FCvmClip {  // cvm_clip: if (v > hi) hi else if (v < lo) lo  (same as FClip when lo <= hi)
  int32_t lo, hi;
  __device__ int32_t operator()(int32_t v) const { return v > hi ? hi : (v < lo ? lo : v); }
};
struct FRShift { RShift r; __device__ int32_t operator()(int32_t v) const { return apply_rshift(r, v); } };
struct FLShift {
  int32_t lo, hi; int b;
  __device__ int32_t operator()(int32_t v) const {
    int32_t t = (int32_t)((uint32_t)v << b);
    t = t < hi ? t : hi;
    return t > lo ? t : lo;
  }
};
struct FAbs { __device__ int32_t operator()(int32_t v) const { return v < 0 ? wsub(0, v) : v; } };
struct FNeg { __device__ int32_t operator()(int32_t v) const { return wsub(0, v); } };
struct FPrecision {  // smallest i in [1,63] with |v| < 2^i; |INT32_MIN| = 2^31 -> 32
  __device__ int32_t operator()(int32_t v) const {
    uint32_t a = v < 0 ? (uint32_t)0 - (uint32_t)v : (uint32_t)v;
    int bl = 32 - __clz(a);  // bit length, 0 for a == 0
    return bl < 1 ? 1 : bl;
  }
};

template <typename F>
__global__ void __launch_bounds__(256) k_unary_vec(const int4* x, int4* y, int64_t nvec, const int32_t* xt,
                                                   int32_t* yt, int tail, F f) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    int4 v = x[i];
    v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
    y[i] = v;
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail) yt[threadIdx.x] = f(xt[threadIdx.x]);
}

// x and y may be the same buffer (no __restrict__): a thread only touches its own element.
template <typename F>
__global__ void __launch_bounds__(256) k_unary(const int32_t* x, int32_t* y, int64_t n, F f) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) y[i] = f(x[i]);
}

template <typename F>
static int launch_unary(const int32_t* x, int32_t* y, int64_t size, F f, void* stream, const char* name) {
  if (size < 0 || (size > 0 && (!x || !y))) return arg_error(name);
  if (size == 0) return CVMHIP_OK;
  hipStream_t s = as_stream(stream);
  const bool aligned = (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
  if (aligned) {
    const int64_t nvec = size / 4;
    const int tail = (int)(size % 4);
    k_unary_vec<F><<<grid_for(nvec, 256), 256, 0, s>>>((const int4*)x, (int4*)y, nvec, x + nvec * 4,
                                                       y + nvec * 4, tail, f);
  } else {
    k_unary<F><<<grid_for(size, 256), 256, 0, s>>>(x, y, size, f);
  }
  return check_launch(name);
}

// ---------------------------------------------------------------- binary ops
template <int OP>
__device__ __forceinline__ int32_t bfun(int32_t a, int32_t b) {
  if (OP == CVMHIP_ADD) return wadd(a, b);
  if (OP == CVMHIP_SUB) return wsub(a, b);
  if (OP == CVMHIP_MUL) return wmul(a, b);
  if (OP == CVMHIP_MAX) return a > b ? a : b;
  if (OP == CVMHIP_DIV) {
    if (b == 0) return 0;
    if (b == -1) return wsub(0, a);  // also covers INT32_MIN / -1 without trapping
    return a / b;
  }
  return a > b ? 1 : 0;
}

template <int OP>
__global__ void __launch_bounds__(256) k_binary(const int32_t* a, const int32_t* b, int32_t* c, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    c[i] = bfun<OP>(a[i], b[i]);
}

template <int OP>
__global__ void __launch_bounds__(256) k_binary_vec(const int4* a, const int4* b, int4* c, int64_t nvec) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    int4 u = a[i], v = b[i], r;
    r.x = bfun<OP>(u.x, v.x); r.y = bfun<OP>(u.y, v.y); r.z = bfun<OP>(u.z, v.z); r.w = bfun<OP>(u.w, v.w);
    c[i] = r;
  }
}

// one operand is a single element (the reference's fast paths, broadcast.cc:33-36): SCALAR_A selects which
template <int OP, bool SCALAR_A>
__global__ void __launch_bounds__(256) k_binary_scalar_vec(const int4* v, const int32_t* scalar, int4* c, int64_t nvec) {
  const int32_t k = scalar[0];
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    const int4 u = v[i];
    int4 r;
    if (SCALAR_A) { r.x = bfun<OP>(k, u.x); r.y = bfun<OP>(k, u.y); r.z = bfun<OP>(k, u.z); r.w = bfun<OP>(k, u.w); }
    else { r.x = bfun<OP>(u.x, k); r.y = bfun<OP>(u.y, k); r.z = bfun<OP>(u.z, k); r.w = bfun<OP>(u.w, k); }
    c[i] = r;
  }
}

struct BShape {
  int ndim;
  int64_t cdim[CVM_MAXD];     // output extents
  int64_t astride[CVM_MAXD];  // element stride of a per output dim (0 where broadcast)
  int64_t bstride[CVM_MAXD];
};

// amode/bmode: 0 = indexed by strides, 1 = scalar (always element 0), 2 = linear (same index as c)
template <int OP>
__global__ void __launch_bounds__(256) k_broadcast(const int32_t* a, const int32_t* b, int32_t* c, int64_t n,
                                                   BShape sh, int amode, int bmode) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t ai = 0, bi = 0;
    if (amode == 0 || bmode == 0) {
      int64_t t = i;
      for (int d = sh.ndim - 1; d >= 0; --d) {
        const int64_t col = t % sh.cdim[d];
        t /= sh.cdim[d];
        ai += col * sh.astride[d];
        bi += col * sh.bstride[d];
      }
    }
    if (amode == 1) ai = 0; else if (amode == 2) ai = i;
    if (bmode == 1) bi = 0; else if (bmode == 2) bi = i;
    c[i] = bfun<OP>(a[ai], b[bi]);
  }
}

template <int OP>
static int launch_broadcast(const int32_t* a, const int32_t* b, int32_t* c, int64_t n, const BShape& sh,
                            int amode, int bmode, hipStream_t s) {
  if (amode == 2 && bmode == 2) {
    const bool aligned = (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0 && (n % 4) == 0;
    if (aligned)
      k_binary_vec<OP><<<grid_for(n / 4, 256), 256, 0, s>>>((const int4*)a, (const int4*)b, (int4*)c, n / 4);
    else
      k_binary<OP><<<grid_for(n, 256), 256, 0, s>>>(a, b, c, n);
  } else if (amode == 2 && bmode == 1 && (((uintptr_t)a | (uintptr_t)c) & 15) == 0 && (n % 4) == 0) {
    k_binary_scalar_vec<OP, false><<<grid_for(n / 4, 256), 256, 0, s>>>((const int4*)a, b, (int4*)c, n / 4);
  } else if (amode == 1 && bmode == 2 && (((uintptr_t)b | (uintptr_t)c) & 15) == 0 && (n % 4) == 0) {
    k_binary_scalar_vec<OP, true><<<grid_for(n / 4, 256), 256, 0, s>>>((const int4*)b, a, (int4*)c, n / 4);
  } else {
    k_broadcast<OP><<<grid_for(n, 256), 256, 0, s>>>(a, b, c, n, sh, amode, bmode);
  }
  return check_launch("broadcast");
}

// ---------------------------------------------------------------- max_pool2d
// One thread per output element; I is the index type (32-bit whenever the tensors allow it: the three
// divisions per element are what this kernel would otherwise spend most of its time on).
template <typename I>
__global__ void __launch_bounds__(256) k_max_pool(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                  int64_t total, int h, int w, int oh, int ow, int kh, int kw,
                                                  int sh, int sw, int ph, int pw) {
  const I stride = (I)gridDim.x * blockDim.x;
  for (I i = (I)blockIdx.x * blockDim.x + threadIdx.x; i < (I)total; i += stride) {
    const I row = i / (I)ow;
    const int q = (int)(i - row * (I)ow);
    const I nc = row / (I)oh;
    const int p = (int)(row - nc * (I)oh);
    const int32_t* xp = x + (int64_t)nc * h * w;
    int32_t m = INT32_MIN;
    for (int r = 0; r < kh; ++r) {
      const int ih = p * sh + r - ph;
      if (ih < 0 || ih >= h) continue;
      for (int t = 0; t < kw; ++t) {
        const int iw = q * sw + t - pw;
        if (iw < 0 || iw >= w) continue;
        const int32_t v = xp[ih * w + iw];
        m = v > m ? v : m;
      }
    }
    y[i] = m;
  }
}

// 3x3 windows with stride 2 (the pooling layer behind a network's input convolution) on rows whose
// length is a multiple of 4: one thread per pair of adjacent outputs.  The two windows span five input
// columns, four of which are one aligned 16-byte load per row, so a pair costs six loads instead of
// eighteen and a wavefront reads whole contiguous KiBs.  pad_w is 0 or 1.
__global__ void __launch_bounds__(256) k_max_pool_3x3s2(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                        uint32_t total_pairs, int h, int w, int oh, int ow, int ph, int pw) {
  const uint32_t pairs = (uint32_t)(ow + 1) >> 1;
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total_pairs; i += stride) {
    const uint32_t row = i / pairs;
    const int j = (int)(i - row * pairs);
    const uint32_t nc = row / (uint32_t)oh;
    const int p = (int)(row - nc * (uint32_t)oh);
    const int32_t* xp = x + (int64_t)nc * h * w + 4 * j;
    int32_t m0 = INT32_MIN, m1 = INT32_MIN;
    const int extra = pw ? -1 : 4;                 // the fifth column, relative to 4j
    const bool extra_ok = pw ? j > 0 : 4 * j + 4 < w;
    // All six loads are issued before the first is used (rows outside the image read the nearest row inside and
    // are masked afterwards): a load under a condition waits for the one before it.
    int4 vv[3];
    int32_t ee[3];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int ih = 2 * p + r - ph;
      const int64_t at = (int64_t)(ih < 0 ? 0 : (ih < h ? ih : h - 1)) * w;
      vv[r] = *reinterpret_cast<const int4*>(xp + at);
      ee[r] = xp[at + (extra_ok ? extra : 0)];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int ih = 2 * p + r - ph;
      if (ih < 0 || ih >= h) continue;
      const int4 v = vv[r];
      const int32_t e = extra_ok ? ee[r] : INT32_MIN;
      if (pw) {   // windows 4j-1..4j+1 and 4j+1..4j+3
        m0 = max(m0, max(e, max(v.x, v.y)));
        m1 = max(m1, max(v.y, max(v.z, v.w)));
      } else {    // windows 4j..4j+2 and 4j+2..4j+4
        m0 = max(m0, max(v.x, max(v.y, v.z)));
        m1 = max(m1, max(v.z, max(v.w, e)));
      }
    }
    int32_t* yp = y + (int64_t)row * ow + 2 * j;
    yp[0] = m0;
    if (2 * j + 1 < ow) yp[1] = m1;
  }
}

// 2x2 windows with stride 2 and no padding, every window inside the image, rows a multiple of 4 long and an even
// number of outputs per row: one thread per pair of adjacent outputs, two aligned 16-byte loads in flight and one
// 8-byte store, so a wavefront reads and writes whole contiguous KiBs.
__global__ void __launch_bounds__(256) k_max_pool_2x2s2(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                        uint32_t total_pairs, int h, int w, int oh, int ow) {
  const uint32_t pairs = (uint32_t)ow >> 1;
  const uint32_t stride = gridDim.x * blockDim.x;
  for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total_pairs; i += stride) {
    const uint32_t row = i / pairs;
    const int j = (int)(i - row * pairs);
    const uint32_t nc = row / (uint32_t)oh;
    const int p = (int)(row - nc * (uint32_t)oh);
    const int32_t* xp = x + (int64_t)nc * h * w + (int64_t)(2 * p) * w + 4 * j;
    const int4 a = *reinterpret_cast<const int4*>(xp);
    const int4 b = *reinterpret_cast<const int4*>(xp + w);
    int2 o;
    o.x = max(max(a.x, a.y), max(b.x, b.y));
    o.y = max(max(a.z, a.w), max(b.z, b.w));
    *reinterpret_cast<int2*>(y + (int64_t)row * ow + 2 * j) = o;
  }
}

// ---------------------------------------------------------------- reductions
struct RShape {
  int nk, nr;
  int64_t kdim[CVM_MAXD], kstride[CVM_MAXD];  // kept dims (output order)
  int64_t rdim[CVM_MAXD], rstride[CVM_MAXD];  // reduced dims
  int64_t rsize;
  int contiguous;  // reduced dims form one contiguous run of rsize elements
};

template <int OP>
__device__ __forceinline__ int32_t rfun(int32_t acc, int32_t v) {
  return OP == CVMHIP_SUM ? wadd(acc, v) : (acc < v ? v : acc);
}

// One 64-lane wavefront per output element; lanes stride over the reduced
// elements, then a DPP/shuffle tree combines them.  Sum wraps, max is
// order-free, so the tree order does not change the bits.
template <int OP>
__global__ void __launch_bounds__(256) k_reduce_wave(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                     int64_t ksize, RShape sh) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t o = wave; o < ksize; o += nwaves) {
    int64_t base = 0, t = o;
    for (int j = sh.nk - 1; j >= 0; --j) {
      base += (t % sh.kdim[j]) * sh.kstride[j];
      t /= sh.kdim[j];
    }
    // every output has rsize >= 1 contributors; lanes without one carry the
    // first element again for max (idempotent) or 0 for sum.
    const int32_t first = x[base];
    int32_t acc = OP == CVMHIP_SUM ? 0 : first;
    for (int64_t r = lane; r < sh.rsize; r += 64) {
      int64_t off = 0;
      if (sh.contiguous) {
        off = r;
      } else {
        int64_t u = r;
        for (int j = sh.nr - 1; j >= 0; --j) {
          off += (u % sh.rdim[j]) * sh.rstride[j];
          u /= sh.rdim[j];
        }
      }
      acc = rfun<OP>(acc, x[base + off]);
    }
    for (int d = 32; d >= 1; d >>= 1) acc = rfun<OP>(acc, __shfl_xor(acc, d, 64));
    if (lane == 0) y[o] = acc;
  }
}

// Short contiguous runs (the trailing dims are the reduced ones and hold at most a few hundred elements: a
// sum over a 7x7 map, a max over 21 class scores): L lanes per output instead of a whole wavefront, so a
// wavefront finishes 64 / L outputs at a time and neighbouring lanes read neighbouring elements.
template <int OP, int L>
__global__ void __launch_bounds__(256) k_reduce_rows(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                     int64_t ksize, int rsize) {
  const int sub = threadIdx.x % L;
  const int64_t step = ((int64_t)gridDim.x * blockDim.x) / L;
  for (int64_t o = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / L; o < ksize; o += step) {
    const int32_t* row = x + o * rsize;
    int32_t acc = OP == CVMHIP_SUM ? 0 : row[0];
    for (int r = sub; r < rsize; r += L) acc = rfun<OP>(acc, row[r]);
#pragma unroll
    for (int d = L / 2; d >= 1; d >>= 1) acc = rfun<OP>(acc, __shfl_xor(acc, d, 64));
    if (sub == 0) y[o] = acc;
  }
}

// Full reduction starting from 0 (the reference's "no axis" case, reduce.cc:42-47).
template <int OP>
__global__ void __launch_bounds__(1024) k_reduce_all(const int32_t* __restrict__ x, int32_t* __restrict__ y, int64_t n) {
  __shared__ int32_t part[16];
  int32_t acc = 0;
  for (int64_t i = threadIdx.x; i < n; i += blockDim.x) acc = rfun<OP>(acc, x[i]);
  for (int d = 32; d >= 1; d >>= 1) acc = rfun<OP>(acc, __shfl_xor(acc, d, 64));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t t = 0;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t = rfun<OP>(t, part[i]);
    y[0] = t;
  }
}

// ---------------------------------------------------------------- remap copy
// y[i] = x[ sum_j ((begin_j + ((col_j / div_j) % mod_j) * step_j) * xstride_j) ]
struct Remap {
  int ndim;
  int64_t ydim[CVM_MAXD];
  int64_t div[CVM_MAXD], mod[CVM_MAXD], begin[CVM_MAXD], step[CVM_MAXD], xstride[CVM_MAXD];
};

__global__ void __launch_bounds__(256) k_remap(const int32_t* __restrict__ x, int32_t* __restrict__ y, int64_t n, Remap m) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t t = i, src = 0;
    for (int j = m.ndim - 1; j >= 0; --j) {
      const int64_t col = t % m.ydim[j];
      t /= m.ydim[j];
      src += (m.begin[j] + ((col / m.div[j]) % m.mod[j]) * m.step[j]) * m.xstride[j];
    }
    y[i] = x[src];
  }
}

static void remap_identity(Remap* m, const int64_t* xshape, const int64_t* yshape, int ndim) {
  m->ndim = ndim;
  int64_t st = 1;
  for (int j = ndim - 1; j >= 0; --j) {
    m->ydim[j] = yshape[j];
    m->div[j] = 1;
    m->mod[j] = INT64_MAX;
    m->begin[j] = 0;
    m->step[j] = 1;
    m->xstride[j] = st;
    st *= xshape[j];
  }
}

static int64_t prod(const int64_t* s, int n) {
  int64_t p = 1;
  for (int i = 0; i < n; ++i) p *= s[i];
  return p;
}

static int launch_remap(const int32_t* x, int32_t* y, const Remap& m, void* stream, const char* name) {
  const int64_t n = prod(m.ydim, m.ndim);
  if (n == 0) return CVMHIP_OK;
  k_remap<<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(x, y, n, m);
  return check_launch(name);
}

// strided 2-D copy: rows of `row` elements, source pitch xpitch, destination pitch ypitch
__global__ void __launch_bounds__(256) k_copy2d(const int32_t* __restrict__ x, int32_t* __restrict__ y, int64_t rows,
                                                int64_t row, int64_t xpitch, int64_t ypitch) {
  const int64_t n = rows * row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / row, c = i % row;
    y[r * ypitch + c] = x[r * xpitch + c];
  }
}

__global__ void __launch_bounds__(256) k_take_flat(const int32_t* __restrict__ x, const int32_t* __restrict__ idx,
                                                   int32_t* __restrict__ y, int64_t n, int64_t xs) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t j = idx[i] < 0 ? 0 : idx[i];
    if (j > xs - 1) j = xs - 1;
    y[i] = x[j];
  }
}

struct TakeShape {
  int yndim, indim, axis;
  int64_t ydim[CVM_MAXD], xstride[CVM_MAXD], istride[CVM_MAXD];
  int32_t axis_extent;
};

__global__ void __launch_bounds__(256) k_take_axis(const int32_t* __restrict__ x, const int32_t* __restrict__ idx,
                                                   int32_t* __restrict__ y, int64_t n, TakeShape sh) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t t = i, xi = 0, ii = 0;
    for (int j = sh.yndim - 1; j >= 0; --j) {
      const int64_t col = t % sh.ydim[j];
      t /= sh.ydim[j];
      if (sh.axis <= j && j < sh.axis + sh.indim) ii += col * sh.istride[j - sh.axis];
      else xi += col * sh.xstride[j < sh.axis ? j : j - sh.indim + 1];
    }
    int32_t v = idx[ii] < 0 ? 0 : idx[ii];
    if (v > sh.axis_extent - 1) v = sh.axis_extent - 1;
    y[i] = x[xi + (int64_t)v * sh.xstride[sh.axis]];
  }
}

__global__ void __launch_bounds__(256) k_where_same(const int32_t* c, const int32_t* x, const int32_t* y, int32_t* o, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) o[i] = c[i] == 0 ? y[i] : x[i];
}

// 1-D condition: the reference copies `row` BYTES of each selected row (ops.cc:1071),
// the rest of the output row keeps whatever it held.
__global__ void __launch_bounds__(256) k_where_rows(const int32_t* c, const uint8_t* x, const uint8_t* y, uint8_t* o,
                                                    int64_t rows, int64_t row) {
  const int64_t n = rows * row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t r = i / row, b = i % row;
    const int64_t off = r * row * 4 + b;
    o[off] = c[r] == 0 ? y[off] : x[off];
  }
}

}  // namespace cvmhip

using namespace cvmhip;

extern "C" {

const char* cvmhip_last_error(void) { return cvmhip::g_err; }

int cvmhip_relu(const int32_t* x, int32_t* y, int64_t size, void* stream) {
  return launch_unary(x, y, size, FRelu(), stream, "relu");
}

int cvmhip_cvm_clip(const int32_t* x, int32_t* y, int64_t size, int precision, void* stream) {
  if (precision < 1 || precision > 32) return arg_error("cvm_clip.precision");
  FCvmClip f;
  prec_range(precision, &f.lo, &f.hi);
  return launch_unary(x, y, size, f, stream, "cvm_clip");
}

int cvmhip_cvm_right_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit, void* stream) {
  if (precision < 1 || precision > 32) return arg_error("cvm_right_shift.precision");
  if (shift_bit < 1 || shift_bit > 32) return arg_error("cvm_right_shift.shift_bit");
  FRShift f;
  f.r = make_rshift(precision, shift_bit);
  return launch_unary(x, y, size, f, stream, "cvm_right_shift");
}

int cvmhip_cvm_left_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit, void* stream) {
  if (precision < 1 || precision > 32) return arg_error("cvm_left_shift.precision");
  if (shift_bit < 1 || shift_bit > 32) return arg_error("cvm_left_shift.shift_bit");
  FLShift f;
  prec_range(precision, &f.lo, &f.hi);
  f.b = shift_bit & 31;
  return launch_unary(x, y, size, f, stream, "cvm_left_shift");
}

int cvmhip_clip(const int32_t* x, int32_t* y, int64_t size, int32_t a_min, int32_t a_max, void* stream) {
  FClip f;
  f.lo = a_min;
  f.hi = a_max;
  return launch_unary(x, y, size, f, stream, "clip");
}

int cvmhip_abs(const int32_t* x, int32_t* y, int64_t size, void* stream) {
  return launch_unary(x, y, size, FAbs(), stream, "abs");
}

int cvmhip_negative(const int32_t* x, int32_t* y, int64_t size, void* stream) {
  return launch_unary(x, y, size, FNeg(), stream, "negative");
}

int cvmhip_cvm_precision(const int32_t* x, int32_t* y, int64_t size, void* stream) {
  return launch_unary(x, y, size, FPrecision(), stream, "cvm_precision");
}

int cvmhip_elemwise(int op, const int32_t* a, const int32_t* b, int32_t* c, int64_t size, void* stream) {
  if (op != CVMHIP_ADD && op != CVMHIP_SUB) return arg_error("elemwise.op");
  if (size < 0 || (size > 0 && (!a || !b || !c))) return arg_error("elemwise");
  if (size == 0) return CVMHIP_OK;
  BShape sh;
  sh.ndim = 0;
  hipStream_t s = as_stream(stream);
  // in-place (c == a or c == b) is safe: each thread reads its element pair before writing
  return op == CVMHIP_ADD ? launch_broadcast<CVMHIP_ADD>(a, b, c, size, sh, 2, 2, s)
                          : launch_broadcast<CVMHIP_SUB>(a, b, c, size, sh, 2, 2, s);
}

int cvmhip_broadcast(int op, const int32_t* a, const int64_t* ashape, int andim,
                     const int32_t* b, const int64_t* bshape, int bndim,
                     int32_t* c, const int64_t* cshape, int cndim, void* stream) {
  if (op < CVMHIP_ADD || op > CVMHIP_GREATER) return arg_error("broadcast.op");
  if (andim < 1 || bndim < 1 || cndim < 1 || andim > CVM_MAXD || bndim > CVM_MAXD || cndim > CVM_MAXD ||
      andim > cndim || bndim > cndim)
    return arg_error("broadcast.ndim");
  const int64_t as = prod(ashape, andim), bs = prod(bshape, bndim), cs = prod(cshape, cndim);
  if (cs == 0) return CVMHIP_OK;
  BShape sh;
  sh.ndim = cndim;
  int64_t ast = 1, bst = 1;
  for (int d = cndim - 1; d >= 0; --d) {
    sh.cdim[d] = cshape[d];
    const int ad = d - (cndim - andim), bd = d - (cndim - bndim);
    const int64_t ae = ad >= 0 ? ashape[ad] : 1, be = bd >= 0 ? bshape[bd] : 1;
    if ((ae != 1 && ae != cshape[d]) || (be != 1 && be != cshape[d])) return arg_error("broadcast.shape");
    sh.astride[d] = ae == 1 ? 0 : ast;
    sh.bstride[d] = be == 1 ? 0 : bst;
    ast *= ae;
    bst *= be;
  }
  // the reference's fast paths (broadcast.cc:33-36): a one-element operand pairs
  // with the other operand read linearly
  int amode = 0, bmode = 0;
  if (as == 1) { amode = 1; bmode = 2; }
  else if (bs == 1) { amode = 2; bmode = 1; }
  else {
    if (as == cs) amode = 2;
    if (bs == cs) bmode = 2;
  }
  hipStream_t s = as_stream(stream);
  switch (op) {
    case CVMHIP_ADD: return launch_broadcast<CVMHIP_ADD>(a, b, c, cs, sh, amode, bmode, s);
    case CVMHIP_SUB: return launch_broadcast<CVMHIP_SUB>(a, b, c, cs, sh, amode, bmode, s);
    case CVMHIP_MUL: return launch_broadcast<CVMHIP_MUL>(a, b, c, cs, sh, amode, bmode, s);
    case CVMHIP_MAX: return launch_broadcast<CVMHIP_MAX>(a, b, c, cs, sh, amode, bmode, s);
    case CVMHIP_DIV: return launch_broadcast<CVMHIP_DIV>(a, b, c, cs, sh, amode, bmode, s);
    default: return launch_broadcast<CVMHIP_GREATER>(a, b, c, cs, sh, amode, bmode, s);
  }
}

int cvmhip_max_pool2d(const int32_t* x, int32_t* y, int n, int c, int h, int w,
                      int oh, int ow, int kh, int kw, int stride_h, int stride_w,
                      int pad_h, int pad_w, void* stream) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || oh < 1 || ow < 1 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
      pad_h < 0 || pad_w < 0)
    return arg_error("max_pool2d");
  const int64_t total = (int64_t)n * c * oh * ow;
  // (the output extent is the caller's: with ceil_mode a last window may start past the row, which only the general kernel handles)
  if (kh == 3 && kw == 3 && stride_h == 2 && stride_w == 2 && pad_w <= 1 && (w & 3) == 0 && w >= 4 && ((ow + 1) / 2) * 4 <= w &&
      (((uintptr_t)x) & 15) == 0 && total < INT32_MAX && (int64_t)n * c * h * w < ((int64_t)1 << 40)) {
    const int64_t pairs = (int64_t)n * c * oh * ((ow + 1) / 2);
    k_max_pool_3x3s2<<<grid_for(pairs, 256, 256 * 64), 256, 0, as_stream(stream)>>>(x, y, (uint32_t)pairs, h, w, oh, ow, pad_h, pad_w);
    return check_launch("max_pool2d");
  }
  if (kh == 2 && kw == 2 && stride_h == 2 && stride_w == 2 && pad_h == 0 && pad_w == 0 && (w & 3) == 0 && (ow & 1) == 0 &&
      2 * ow <= w && 2 * oh <= h && (((uintptr_t)x) & 15) == 0 && (((uintptr_t)y) & 7) == 0 && total < INT32_MAX &&
      (int64_t)n * c * h * w < ((int64_t)1 << 40)) {
    const int64_t pairs = total / 2;
    k_max_pool_2x2s2<<<grid_for(pairs, 256, 256 * 64), 256, 0, as_stream(stream)>>>(x, y, (uint32_t)pairs, h, w, oh, ow);
    return check_launch("max_pool2d");
  }
  const unsigned grid = grid_for(total, 256, 256 * 64);
  if (total + (int64_t)grid * 256 < INT32_MAX && (int64_t)h * w < INT32_MAX)
    k_max_pool<uint32_t><<<grid, 256, 0, as_stream(stream)>>>(x, y, total, h, w, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w);
  else
    k_max_pool<int64_t><<<grid, 256, 0, as_stream(stream)>>>(x, y, total, h, w, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w);
  return check_launch("max_pool2d");
}

int cvmhip_reduce(int op, const int32_t* x, const int64_t* xshape, int ndim,
                  int32_t* y, int64_t ysize, const int64_t* axes, int naxes, int exclude, void* stream) {
  if (op != CVMHIP_SUM && op != CVMHIP_RMAX) return arg_error("reduce.op");
  if (ndim < 1 || ndim > CVM_MAXD || naxes < 0 || naxes > CVM_MAXD) return arg_error("reduce.ndim");
  bool listed[CVM_MAXD] = {false};
  for (int i = 0; i < naxes; ++i) {
    int64_t a = axes[i] < 0 ? axes[i] + ndim : axes[i];
    if (a < 0 || a >= ndim) return arg_error("reduce.axis");
    listed[a] = true;
  }
  bool red[CVM_MAXD];
  int nreal = 0;
  for (int d = 0; d < ndim; ++d) {
    red[d] = exclude ? !listed[d] : listed[d];
    nreal += red[d];
  }
  const int64_t xsize = prod(xshape, ndim);
  hipStream_t s = as_stream(stream);
  if (exclude && nreal == 0) return cvmhip_copy(x, y, xsize, stream);
  if (nreal == 0) {
    if (op == CVMHIP_SUM) k_reduce_all<CVMHIP_SUM><<<1, 1024, 0, s>>>(x, y, xsize);
    else k_reduce_all<CVMHIP_RMAX><<<1, 1024, 0, s>>>(x, y, xsize);
    return check_launch("reduce_all");
  }
  int64_t stride[CVM_MAXD];
  stride[ndim - 1] = 1;
  for (int d = ndim - 2; d >= 0; --d) stride[d] = stride[d + 1] * xshape[d + 1];
  RShape sh;
  sh.nk = sh.nr = 0;
  sh.rsize = 1;
  int64_t ksize = 1;
  for (int d = 0; d < ndim; ++d) {
    if (red[d]) { sh.rdim[sh.nr] = xshape[d]; sh.rstride[sh.nr++] = stride[d]; sh.rsize *= xshape[d]; }
    else { sh.kdim[sh.nk] = xshape[d]; sh.kstride[sh.nk++] = stride[d]; ksize *= xshape[d]; }
  }
  if (ksize != ysize) return arg_error("reduce.ysize");
  // contiguous run: the reduced dims are the trailing dims
  sh.contiguous = 1;
  for (int d = ndim - nreal; d < ndim; ++d) if (!red[d]) sh.contiguous = 0;
  if (sh.contiguous && sh.rsize <= 512) {
    if (sh.rsize <= 64) {
      const unsigned grid = grid_for(ksize * 8, 256);
      if (op == CVMHIP_SUM) k_reduce_rows<CVMHIP_SUM, 8><<<grid, 256, 0, s>>>(x, y, ksize, (int)sh.rsize);
      else k_reduce_rows<CVMHIP_RMAX, 8><<<grid, 256, 0, s>>>(x, y, ksize, (int)sh.rsize);
    } else {
      const unsigned grid = grid_for(ksize * 32, 256);
      if (op == CVMHIP_SUM) k_reduce_rows<CVMHIP_SUM, 32><<<grid, 256, 0, s>>>(x, y, ksize, (int)sh.rsize);
      else k_reduce_rows<CVMHIP_RMAX, 32><<<grid, 256, 0, s>>>(x, y, ksize, (int)sh.rsize);
    }
    return check_launch("reduce");
  }
  const int64_t threads = ksize * 64;
  if (op == CVMHIP_SUM) k_reduce_wave<CVMHIP_SUM><<<grid_for(threads, 256), 256, 0, s>>>(x, y, ksize, sh);
  else k_reduce_wave<CVMHIP_RMAX><<<grid_for(threads, 256), 256, 0, s>>>(x, y, ksize, sh);
  return check_launch("reduce");
}

int cvmhip_copy(const int32_t* x, int32_t* y, int64_t size, void* stream) {
  if (size < 0) return arg_error("copy.size");
  if (size == 0 || x == y) return CVMHIP_OK;
  hipError_t e = hipMemcpyAsync(y, x, (size_t)size * 4, hipMemcpyDeviceToDevice, as_stream(stream));
  if (e != hipSuccess) { set_error("copy: %s", hipGetErrorString(e)); return CVMHIP_ERR_RUNTIME; }
  return CVMHIP_OK;
}

int cvmhip_concatenate(const int32_t* const* inputs, const int64_t* const* ishapes, int ninputs,
                       int ndim, int axis, int32_t* y, const int64_t* yshape, void* stream) {
  if (ninputs < 1 || ndim < 1 || ndim > CVM_MAXD) return arg_error("concatenate");
  if (axis < 0) axis += ndim;
  if (axis < 0 || axis >= ndim) return arg_error("concatenate.axis");
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= yshape[i];
  for (int i = axis + 1; i < ndim; ++i) inner *= yshape[i];
  const int64_t yrow = yshape[axis] * inner;
  int64_t start = 0;
  for (int m = 0; m < ninputs; ++m) {
    const int64_t xrow = ishapes[m][axis] * inner;
    if (start + xrow > yrow) return arg_error("concatenate.shape");
    const int64_t n = outer * xrow;
    if (n > 0 && inputs[m] != nullptr) {  // a null input: that slice of y is already in place
      k_copy2d<<<grid_for(n, 256), 256, 0, as_stream(stream)>>>(inputs[m], y + start, outer, xrow, xrow, yrow);
      int rc = check_launch("concatenate");
      if (rc) return rc;
    }
    start += xrow;
  }
  return CVMHIP_OK;
}

// Batched 2-D transpose through LDS: x [B][R][C] -> y [B][C][R], both sides read and written in whole
// 128-byte rows of a 32 x 32 tile (the padding column keeps the transposed LDS reads free of bank conflicts).
// Covers every permutation that moves a trailing group of dims in front of the group before it, e.g. the
// NCHW -> NHWC transpose (0, 2, 3, 1) of a detection head and the reference's fast path (1, 2, 0) (ops.cc:759-766).
__global__ void __launch_bounds__(256) k_transpose2d(const int32_t* __restrict__ x, int32_t* __restrict__ y,
                                                     int64_t rows, int64_t cols, int64_t tiles_r, int64_t tiles_c) {
  __shared__ int32_t tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8 threads
  const int64_t per_batch = tiles_r * tiles_c;
  const int64_t b = blockIdx.x / per_batch;
  const int64_t t = blockIdx.x - b * per_batch;
  const int64_t tr = t / tiles_c, tc = t - tr * tiles_c;
  const int32_t* xb = x + b * rows * cols;
  int32_t* yb = y + b * rows * cols;
#pragma unroll
  for (int i = 0; i < 32; i += 8) {
    const int64_t r = tr * 32 + ty + i, c = tc * 32 + tx;
    if (r < rows && c < cols) tile[ty + i][tx] = xb[r * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 32; i += 8) {
    const int64_t c = tc * 32 + ty + i, r = tr * 32 + tx;
    if (r < rows && c < cols) yb[c * rows + r] = tile[tx][ty + i];
  }
}

int cvmhip_transpose(const int32_t* x, const int64_t* xshape, int ndim,
                     const int64_t* axes, int naxes, int32_t* y, void* stream) {
  if (ndim < 1 || ndim > CVM_MAXD || (naxes != 0 && naxes != ndim)) return arg_error("transpose");
  int64_t xstride[CVM_MAXD];
  xstride[ndim - 1] = 1;
  for (int d = ndim - 2; d >= 0; --d) xstride[d] = xstride[d + 1] * xshape[d + 1];
  Remap m;
  m.ndim = ndim;
  for (int j = 0; j < ndim; ++j) {
    int64_t p = naxes ? (axes[j] < 0 ? axes[j] + ndim : axes[j]) : ndim - 1 - j;
    if (p < 0 || p >= ndim) return arg_error("transpose.axes");
    m.ydim[j] = xshape[p];
    m.div[j] = 1; m.mod[j] = INT64_MAX; m.begin[j] = 0; m.step[j] = 1;
    m.xstride[j] = xstride[p];
  }
  // a prefix kept in place, then the trailing group of dims moved in front of the group before it?
  {
    int64_t perm[CVM_MAXD];
    for (int j = 0; j < ndim; ++j) perm[j] = naxes ? (axes[j] < 0 ? axes[j] + ndim : axes[j]) : ndim - 1 - j;
    int b = 0;
    while (b < ndim && perm[b] == b) ++b;
    if (b < ndim) {
      const int mid = (int)perm[b];            // first dim of the trailing group
      bool ok = mid > b;
      for (int j = b; ok && j < ndim; ++j) ok = perm[j] == (j - b < ndim - mid ? mid + (j - b) : b + (j - b - (ndim - mid)));
      if (ok) {
        int64_t batch = 1, rows = 1, cols = 1;
        for (int d = 0; d < b; ++d) batch *= xshape[d];
        for (int d = b; d < mid; ++d) rows *= xshape[d];
        for (int d = mid; d < ndim; ++d) cols *= xshape[d];
        const int64_t tiles_r = (rows + 31) / 32, tiles_c = (cols + 31) / 32;
        const int64_t blocks = batch * tiles_r * tiles_c;
        if (rows > 1 && cols > 1 && blocks > 0 && blocks < 0x7fffffff) {
          k_transpose2d<<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(x, y, rows, cols, tiles_r, tiles_c);
          return check_launch("transpose");
        }
      }
    }
  }
  return launch_remap(x, y, m, stream, "transpose");
}

int cvmhip_strided_slice(const int32_t* x, const int64_t* xshape, int ndim,
                         const int64_t* begin, int nbegin, const int64_t* stride, int nstride,
                         int32_t* y, const int64_t* yshape, void* stream) {
  if (ndim < 1 || ndim > CVM_MAXD) return arg_error("strided_slice");
  Remap m;
  remap_identity(&m, xshape, yshape, ndim);
  for (int i = 0; i < ndim; ++i) {
    const int64_t sv = i < nstride ? stride[i] : 1;
    if (sv == 0) return arg_error("strided_slice.stride");
    const int64_t lo = sv < 0 ? -1 : 0, hi = sv < 0 ? xshape[i] - 1 : xshape[i];
    int64_t b = i < nbegin ? begin[i] : 0;
    if (b < 0) b += xshape[i];
    if (b < lo) b = lo;
    if (b > hi) b = hi;
    // last element read on this axis must stay inside x
    const int64_t last = b + (yshape[i] - 1) * sv;
    if (yshape[i] > 0 && (b < 0 || b >= xshape[i] || last < 0 || last >= xshape[i])) return arg_error("strided_slice.range");
    m.begin[i] = b;
    m.step[i] = sv;
  }
  return launch_remap(x, y, m, stream, "strided_slice");
}

int cvmhip_slice_like(const int32_t* x, const int64_t* xshape, int ndim,
                      int32_t* y, const int64_t* yshape, void* stream) {
  if (ndim < 1 || ndim > CVM_MAXD) return arg_error("slice_like");
  for (int i = 0; i < ndim; ++i) if (yshape[i] > xshape[i]) return arg_error("slice_like.shape");
  Remap m;
  remap_identity(&m, xshape, yshape, ndim);
  return launch_remap(x, y, m, stream, "slice_like");
}

int cvmhip_repeat(const int32_t* x, const int64_t* xshape, int32_t* y, const int64_t* yshape,
                  int ndim, int axis, int repeats, void* stream) {
  if (ndim < 1 || ndim > CVM_MAXD || repeats < 1) return arg_error("repeat");
  if (axis < 0) axis += ndim;
  if (axis < 0 || axis >= ndim) return arg_error("repeat.axis");
  for (int i = 0; i < ndim; ++i)
    if (yshape[i] != xshape[i] * (i == axis ? repeats : 1)) return arg_error("repeat.shape");
  Remap m;
  remap_identity(&m, xshape, yshape, ndim);
  m.div[axis] = repeats;
  return launch_remap(x, y, m, stream, "repeat");
}

int cvmhip_tile(const int32_t* x, const int64_t* xshape, int xndim,
                int32_t* y, const int64_t* yshape, int yndim, void* stream) {
  if (xndim < 1 || yndim < xndim || yndim > CVM_MAXD) return arg_error("tile");
  const int lead = yndim - xndim;
  Remap m;
  m.ndim = yndim;
  int64_t st = 1;
  for (int j = yndim - 1; j >= 0; --j) {
    m.ydim[j] = yshape[j];
    m.div[j] = 1; m.begin[j] = 0; m.step[j] = 1;
    if (j >= lead) {
      m.mod[j] = xshape[j - lead];
      m.xstride[j] = st;
      st *= xshape[j - lead];
    } else {
      m.mod[j] = 1;  // leading output dims replicate the whole block
      m.xstride[j] = 0;
    }
  }
  return launch_remap(x, y, m, stream, "tile");
}

int cvmhip_upsampling(const int32_t* x, int32_t* y, int n, int c, int h, int w, int scale, void* stream) {
  if (n < 1 || c < 1 || h < 1 || w < 1 || scale < 1) return arg_error("upsampling");
  const int64_t xs[4] = {n, c, h, w}, ys[4] = {n, c, (int64_t)h * scale, (int64_t)w * scale};
  Remap m;
  remap_identity(&m, xs, ys, 4);
  m.div[2] = m.div[3] = scale;
  return launch_remap(x, y, m, stream, "upsampling");
}

int cvmhip_take(const int32_t* x, const int64_t* xshape, int xndim,
                const int32_t* indices, const int64_t* ishape, int indim,
                int32_t* y, const int64_t* yshape, int yndim, int has_axis, int axis, void* stream) {
  if (xndim < 1 || xndim > CVM_MAXD || indim < 1 || indim > CVM_MAXD || yndim < 1 || yndim > CVM_MAXD)
    return arg_error("take.ndim");
  const int64_t n = prod(yshape, yndim);
  if (n == 0) return CVMHIP_OK;
  hipStream_t s = as_stream(stream);
  if (!has_axis) {
    if (n != prod(ishape, indim)) return arg_error("take.shape");
    k_take_flat<<<grid_for(n, 256), 256, 0, s>>>(x, indices, y, n, prod(xshape, xndim));
    return check_launch("take");
  }
  if (axis < 0) axis += xndim;
  if (axis < 0 || axis >= xndim || yndim != xndim - 1 + indim) return arg_error("take.axis");
  TakeShape sh;
  sh.yndim = yndim; sh.indim = indim; sh.axis = axis;
  sh.axis_extent = (int32_t)xshape[axis];
  for (int j = 0; j < yndim; ++j) sh.ydim[j] = yshape[j];
  sh.xstride[xndim - 1] = 1;
  for (int i = xndim - 2; i >= 0; --i) sh.xstride[i] = sh.xstride[i + 1] * xshape[i + 1];
  sh.istride[indim - 1] = 1;
  for (int i = indim - 2; i >= 0; --i) sh.istride[i] = sh.istride[i + 1] * ishape[i + 1];
  k_take_axis<<<grid_for(n, 256), 256, 0, s>>>(x, indices, y, n, sh);
  return check_launch("take");
}

int cvmhip_where(const int32_t* cond, const int32_t* x, const int32_t* y, int32_t* out,
                 const int64_t* oshape, int ndim, int same_shape, void* stream) {
  if (ndim < 1 || ndim > CVM_MAXD) return arg_error("where");
  hipStream_t s = as_stream(stream);
  if (same_shape) {
    const int64_t n = prod(oshape, ndim);
    if (n == 0) return CVMHIP_OK;
    k_where_same<<<grid_for(n, 256), 256, 0, s>>>(cond, x, y, out, n);
  } else {
    const int64_t row = prod(oshape + 1, ndim - 1);
    if (row * oshape[0] == 0) return CVMHIP_OK;
    k_where_rows<<<grid_for(row * oshape[0], 256), 256, 0, s>>>(cond, (const uint8_t*)x, (const uint8_t*)y,
                                                               (uint8_t*)out, oshape[0], row);
  }
  return check_launch("where");
}

}  // extern "C"
