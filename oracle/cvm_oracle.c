/*
 * TEST INFRASTRUCTURE ONLY -- see cvm_oracle.h.  CPU restatement of the
 * reference CVM CPU operators.  Integer arithmetic wraps modulo 2^32 exactly
 * like the reference's int32 accumulators do on x86 (-fwrapv semantics are
 * obtained by computing in uint32_t).
 */
#include "cvm_oracle.h"

#include <stdlib.h>
#include <string.h>

#define MAXD 6

static inline int32_t wadd(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
static inline int32_t wsub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
static inline int32_t wmul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }

static int64_t prod(const int64_t* s, int n) {
  int64_t p = 1;
  for (int i = 0; i < n; ++i) p *= s[i];
  return p;
}

/* ------------------------------------------------------------------ conv2d */
/* groups == 1 (ops.cc:425-452): filter and input are narrowed with
 * static_cast<int8_t> (ops.cc:234,431), products accumulate in int32, bias is
 * added last.  Here the col matrix is built for the whole batch at once and the
 * product is accumulated row-by-row (i-k-j order) -- any order gives the same
 * bits because the accumulation wraps.  groups > 1 (ops.cc:333-366): direct
 * loops on the int32 values, no narrowing. */
int cvmo_conv2d(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                int n, int ic, int h, int wd, int oc, int kh, int kw,
                int stride_h, int stride_w, int pad_h, int pad_w,
                int dil_h, int dil_w, int groups) {
  if (groups < 1 || ic % groups || oc % groups || stride_h < 1 || stride_w < 1) return 1;
  const int oh = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  const int ow = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  if (oh <= 0 || ow <= 0) return 1;
  const int64_t ohw = (int64_t)oh * ow;
  if (groups > 1) {
    const int icg = ic / groups, ocg = oc / groups;
#pragma omp parallel for collapse(2)
    for (int b = 0; b < n; ++b)
      for (int o = 0; o < oc; ++o) {
        const int c0 = (o / ocg) * icg;
        for (int p = 0; p < oh; ++p)
          for (int q = 0; q < ow; ++q) {
            int32_t acc = 0;
            for (int c = 0; c < icg; ++c)
              for (int r = 0; r < kh; ++r) {
                const int ih = p * stride_h + r * dil_h - pad_h;
                if (ih < 0 || ih >= h) continue;
                for (int s = 0; s < kw; ++s) {
                  const int iw = q * stride_w + s * dil_w - pad_w;
                  if (iw < 0 || iw >= wd) continue;
                  acc = wadd(acc, wmul(x[(((int64_t)b * ic + c0 + c) * h + ih) * wd + iw],
                                       w[(((int64_t)o * icg + c) * kh + r) * kw + s]));
                }
              }
            y[((int64_t)b * oc + o) * ohw + (int64_t)p * ow + q] = wadd(acc, bias ? bias[o] : 0);
          }
      }
    return 0;
  }
  const int64_t K = (int64_t)ic * kh * kw;
  int8_t* w8 = (int8_t*)malloc((size_t)oc * K);
  int8_t* col = (int8_t*)malloc((size_t)K * ohw);
  if (!w8 || !col) { free(w8); free(col); return 2; }
  for (int64_t i = 0; i < (int64_t)oc * K; ++i) w8[i] = (int8_t)w[i];
  for (int b = 0; b < n; ++b) {
    const int32_t* xb = x + (int64_t)b * ic * h * wd;
#pragma omp parallel for
    for (int64_t kk = 0; kk < K; ++kk) {
      const int c = (int)(kk / (kh * kw)), r = (int)((kk / kw) % kh), s = (int)(kk % kw);
      int8_t* dst = col + kk * ohw;
      for (int p = 0; p < oh; ++p) {
        const int ih = p * stride_h + r * dil_h - pad_h;
        for (int q = 0; q < ow; ++q) {
          const int iw = q * stride_w + s * dil_w - pad_w;
          int8_t v = 0;
          if (ih >= 0 && ih < h && iw >= 0 && iw < wd)
            v = (int8_t)xb[((int64_t)c * h + ih) * wd + iw];
          dst[(int64_t)p * ow + q] = v;
        }
      }
    }
    int32_t* yb = y + (int64_t)b * oc * ohw;
#pragma omp parallel for
    for (int o = 0; o < oc; ++o) {
      int32_t* row = yb + (int64_t)o * ohw;
      const int32_t b0 = bias ? bias[o] : 0;
      for (int64_t j = 0; j < ohw; ++j) row[j] = 0;
      for (int64_t kk = 0; kk < K; ++kk) {
        const int32_t a = w8[(int64_t)o * K + kk];
        if (a == 0) continue;
        const int8_t* cr = col + kk * ohw;
        for (int64_t j = 0; j < ohw; ++j) row[j] = wadd(row[j], wmul(a, cr[j]));
      }
      for (int64_t j = 0; j < ohw; ++j) row[j] = wadd(row[j], b0);
    }
  }
  free(w8);
  free(col);
  return 0;
}

/* ------------------------------------------------------------------- dense */
/* ops.cc:34-75: Y[m][j] = sum_k X[m][k] * W[j][k] (+ B[j]); int32 operands, no narrowing. */
int cvmo_dense(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
               int m, int k, int n) {
#pragma omp parallel for collapse(2)
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      int32_t acc = 0;
      const int32_t* xr = x + (int64_t)i * k;
      const int32_t* wr = w + (int64_t)j * k;
      for (int t = 0; t < k; ++t) acc = wadd(acc, wmul(xr[t], wr[t]));
      y[(int64_t)i * n + j] = wadd(acc, bias ? bias[j] : 0);
    }
  return 0;
}

/* --------------------------------------------------------------- elementwise */
int cvmo_relu(const int32_t* x, int32_t* y, int64_t size) {
  for (int64_t i = 0; i < size; ++i) y[i] = x[i] < 0 ? 0 : x[i];
  return 0;
}

/* elemwise.cc:100-110: range is +-(2^(p-1) - 1), computed in int64 then narrowed. */
static void prec_range(int precision, int32_t* lo, int32_t* hi) {
  int32_t mn = (int32_t)(-((((int64_t)1) << (precision - 1)) - 1));
  *lo = mn;
  *hi = (int32_t)(-(int64_t)mn);
}

int cvmo_cvm_clip(const int32_t* x, int32_t* y, int64_t size, int precision) {
  if (precision < 1 || precision > 32) return 1;
  int32_t lo, hi;
  prec_range(precision, &lo, &hi);
  for (int64_t i = 0; i < size; ++i) {
    int32_t t = x[i];
    if (t > hi) t = hi; else if (t < lo) t = lo;
    y[i] = t;
  }
  return 0;
}

/* elemwise.cc:128-148.  Four regimes, in the reference's order:
 *   max == 0            -> zeros
 *   b >= 31             -> a >> 31 (no clip)
 *   precision + b >= 32 -> ((a >> (b-1)) + 1) >> 1 (no clip)
 *   otherwise           -> saturate on pre-shifted bounds, else the rounding shift. */
int cvmo_cvm_right_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit) {
  if (precision < 1 || precision > 32 || shift_bit < 1 || shift_bit > 32) return 1;
  int32_t lo, hi;
  prec_range(precision, &lo, &hi);
  const int b = shift_bit;
  if (hi == 0) {
    for (int64_t i = 0; i < size; ++i) y[i] = 0;
  } else if (b >= 31) {
    for (int64_t i = 0; i < size; ++i) y[i] = x[i] >> 31;
  } else if (precision + b >= 32) {
    for (int64_t i = 0; i < size; ++i) y[i] = wadd(x[i] >> (b - 1), 1) >> 1;
  } else {
    const int32_t x_min = (int32_t)((uint32_t)(-2 * hi - 1) << (b - 1));
    const int32_t x_max = (int32_t)((uint32_t)(2 * hi - 1) << (b - 1));
    for (int64_t i = 0; i < size; ++i) {
      const int32_t t = x[i];
      if (t < x_min) y[i] = lo;
      else if (t > x_max) y[i] = hi;
      else y[i] = ((t >> (b - 1)) + 1) >> 1;
    }
  }
  return 0;
}

int cvmo_cvm_left_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit) {
  if (precision < 1 || precision > 32 || shift_bit < 1 || shift_bit > 32) return 1;
  int32_t lo, hi;
  prec_range(precision, &lo, &hi);
  for (int64_t i = 0; i < size; ++i) {
    /* x86 masks the shift count to 5 bits for a 32-bit shl */
    int32_t t = (int32_t)((uint32_t)x[i] << (shift_bit & 31));
    if (t > hi) t = hi;
    if (t < lo) t = lo;
    y[i] = t;
  }
  return 0;
}

int cvmo_clip(const int32_t* x, int32_t* y, int64_t size, int32_t a_min, int32_t a_max) {
  for (int64_t i = 0; i < size; ++i) {
    int32_t t = x[i] < a_max ? x[i] : a_max;   /* min(max, x) */
    y[i] = t > a_min ? t : a_min;              /* max(., min) */
  }
  return 0;
}

int cvmo_elemwise(int op, const int32_t* a, const int32_t* b, int32_t* c, int64_t size) {
  if (op == CVMO_ADD) for (int64_t i = 0; i < size; ++i) c[i] = wadd(a[i], b[i]);
  else if (op == CVMO_SUB) for (int64_t i = 0; i < size; ++i) c[i] = wsub(a[i], b[i]);
  else return 1;
  return 0;
}

int cvmo_abs(const int32_t* x, int32_t* y, int64_t size) {
  for (int64_t i = 0; i < size; ++i) y[i] = x[i] < 0 ? wsub(0, x[i]) : x[i];
  return 0;
}

int cvmo_negative(const int32_t* x, int32_t* y, int64_t size) {
  for (int64_t i = 0; i < size; ++i) y[i] = wsub(0, x[i]);
  return 0;
}

/* ops.cc:531-541: smallest i in [1,63] with |x| < 2^i (|x| in int64). */
int cvmo_cvm_precision(const int32_t* x, int32_t* y, int64_t size) {
  for (int64_t j = 0; j < size; ++j) {
    int64_t v = x[j];
    if (v < 0) v = -v;
    int32_t r = 64;
    for (int i = 1; i < 64; ++i)
      if (v < ((int64_t)1 << i)) { r = i; break; }
    y[j] = r;
  }
  return 0;
}

/* ---------------------------------------------------------------- broadcast */
static inline int32_t bfun(int op, int32_t a, int32_t b) {
  switch (op) {
    case CVMO_ADD: return wadd(a, b);
    case CVMO_SUB: return wsub(a, b);
    case CVMO_MUL: return wmul(a, b);
    case CVMO_MAX: return a > b ? a : b;
    case CVMO_DIV:
      if (b == 0) return 0;
      if (a == INT32_MIN && b == -1) return INT32_MIN; /* idiv would trap; keep defined */
      return a / b;
    default: return a > b;
  }
}

/* broadcast.cc:6-21: right-aligned index of the output position inside an input. */
static int64_t bindex(const int64_t* oshape, int odim, int64_t oidx, const int64_t* ishape, int idim) {
  if (idim == 1 && ishape[0] == 1) return 0;
  int64_t index = 0, mul = 1;
  for (int i = 0; i < idim; ++i) {
    const int d = idim - 1 - i;
    const int64_t ovar = oidx % oshape[d + odim - idim];
    if (ovar < ishape[d]) index += mul * ovar;
    mul *= ishape[d];
    oidx /= oshape[d + odim - idim];
  }
  return index;
}

int cvmo_broadcast(int op, const int32_t* a, const int64_t* ashape, int andim,
                   const int32_t* b, const int64_t* bshape, int bndim,
                   int32_t* c, const int64_t* cshape, int cndim) {
  if (op < 0 || op > CVMO_GREATER) return 1;
  const int64_t as = prod(ashape, andim), bs = prod(bshape, bndim), cs = prod(cshape, cndim);
  if (as == 1) {
    for (int64_t i = 0; i < cs; ++i) c[i] = bfun(op, a[0], b[i]);
  } else if (bs == 1) {
    for (int64_t i = 0; i < cs; ++i) c[i] = bfun(op, a[i], b[0]);
  } else {
#pragma omp parallel for
    for (int64_t i = 0; i < cs; ++i)
      c[i] = bfun(op, a[bindex(cshape, cndim, i, ashape, andim)],
                  b[bindex(cshape, cndim, i, bshape, bndim)]);
  }
  return 0;
}

/* --------------------------------------------------------------- max_pool2d */
int cvmo_max_pool2d(const int32_t* x, int32_t* y, int n, int c, int h, int w,
                    int oh, int ow, int kh, int kw, int stride_h, int stride_w,
                    int pad_h, int pad_w) {
#pragma omp parallel for
  for (int64_t nc = 0; nc < (int64_t)n * c; ++nc) {
    const int32_t* xp = x + nc * h * w;
    int32_t* yp = y + nc * oh * ow;
    for (int p = 0; p < oh; ++p)
      for (int q = 0; q < ow; ++q) {
        int32_t m = INT32_MIN;
        for (int r = 0; r < kh; ++r)
          for (int s = 0; s < kw; ++s) {
            const int ih = p * stride_h + r - pad_h, iw = q * stride_w + s - pad_w;
            if (ih >= 0 && ih < h && iw >= 0 && iw < w) {
              const int32_t v = xp[(int64_t)ih * w + iw];
              if (v > m) m = v;
            }
          }
        yp[(int64_t)p * ow + q] = m;
      }
  }
  return 0;
}

/* ------------------------------------------------------------------- reduce */
/* reduce.cc:34-105.  Three cases: (exclude && no real axis) copies; (no axis,
 * !exclude) folds everything starting from 0; otherwise every output element
 * starts from its first contributing input and folds the rest. */
int cvmo_reduce(int op, const int32_t* x, const int64_t* xshape, int ndim,
                int32_t* y, int64_t ysize, const int64_t* axes, int naxes, int exclude) {
  if (ndim < 1 || ndim > MAXD || naxes > MAXD) return 1;
  int red[MAXD] = {0};
  int listed[MAXD] = {0};
  for (int i = 0; i < naxes; ++i) {
    int64_t a = axes[i] < 0 ? axes[i] + ndim : axes[i];
    if (a < 0 || a >= ndim) return 1;
    listed[a] = 1;
  }
  int nreal = 0;
  for (int d = 0; d < ndim; ++d) {
    red[d] = exclude ? !listed[d] : listed[d];
    nreal += red[d];
  }
  const int64_t xsize = prod(xshape, ndim);
  if (exclude && nreal == 0) {
    memcpy(y, x, (size_t)xsize * 4);
    return 0;
  }
  if (nreal == 0) {
    int32_t t = 0;
    for (int64_t i = 0; i < xsize; ++i) {
      if (op == CVMO_SUM) t = wadd(t, x[i]); else if (t < x[i]) t = x[i];
    }
    y[0] = t;
    return 0;
  }
  int64_t stride[MAXD];
  stride[ndim - 1] = 1;
  for (int d = ndim - 2; d >= 0; --d) stride[d] = stride[d + 1] * xshape[d + 1];
  int kd[MAXD], nk = 0, rd[MAXD], nr = 0;
  int64_t rsize = 1, ksize = 1;
  for (int d = 0; d < ndim; ++d) {
    if (red[d]) { rd[nr++] = d; rsize *= xshape[d]; }
    else { kd[nk++] = d; ksize *= xshape[d]; }
  }
  if (ksize != ysize) return 1;
#pragma omp parallel for
  for (int64_t o = 0; o < ksize; ++o) {
    int64_t base = 0, t = o;
    for (int j = nk - 1; j >= 0; --j) {
      base += (t % xshape[kd[j]]) * stride[kd[j]];
      t /= xshape[kd[j]];
    }
    int32_t acc = x[base];
    for (int64_t r = 1; r < rsize; ++r) {
      int64_t off = 0, u = r;
      for (int j = nr - 1; j >= 0; --j) {
        off += (u % xshape[rd[j]]) * stride[rd[j]];
        u /= xshape[rd[j]];
      }
      const int32_t v = x[base + off];
      if (op == CVMO_SUM) acc = wadd(acc, v); else if (acc < v) acc = v;
    }
    y[o] = acc;
  }
  return 0;
}

/* -------------------------------------------------------- index-remap copies */
int cvmo_concatenate(const int32_t* const* inputs, const int64_t* const* ishapes, int ninputs,
                     int ndim, int axis, int32_t* y, const int64_t* yshape) {
  if (axis < 0) axis += ndim;
  if (axis < 0 || axis >= ndim) return 1;
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= yshape[i];
  for (int i = axis + 1; i < ndim; ++i) inner *= yshape[i];
  const int64_t yrow = yshape[axis] * inner;
  int64_t start = 0;
  for (int m = 0; m < ninputs; ++m) {
    const int64_t xrow = ishapes[m][axis] * inner;
    for (int64_t o = 0; o < outer; ++o)
      memcpy(y + o * yrow + start, inputs[m] + o * xrow, (size_t)xrow * 4);
    start += xrow;
  }
  return 0;
}

int cvmo_transpose(const int32_t* x, const int64_t* xshape, int ndim,
                   const int64_t* axes, int naxes, int32_t* y) {
  if (ndim < 1 || ndim > MAXD || (naxes != 0 && naxes != ndim)) return 1;
  int64_t perm[MAXD], yshape[MAXD], xstride[MAXD];
  for (int j = 0; j < ndim; ++j) {
    perm[j] = naxes ? (axes[j] < 0 ? axes[j] + ndim : axes[j]) : ndim - 1 - j;
    if (perm[j] < 0 || perm[j] >= ndim) return 1;
    yshape[j] = xshape[perm[j]];
  }
  xstride[ndim - 1] = 1;
  for (int d = ndim - 2; d >= 0; --d) xstride[d] = xstride[d + 1] * xshape[d + 1];
  const int64_t size = prod(xshape, ndim);
#pragma omp parallel for
  for (int64_t i = 0; i < size; ++i) {
    int64_t t = i, src = 0;
    for (int j = ndim - 1; j >= 0; --j) {
      src += (t % yshape[j]) * xstride[perm[j]];
      t /= yshape[j];
    }
    y[i] = x[src];
  }
  return 0;
}

int cvmo_strided_slice(const int32_t* x, const int64_t* xshape, int ndim,
                       const int64_t* begin, int nbegin, const int64_t* stride, int nstride,
                       int32_t* y, const int64_t* yshape) {
  if (ndim < 1 || ndim > MAXD) return 1;
  int64_t bv[MAXD], sv[MAXD];
  for (int i = 0; i < ndim; ++i) {
    bv[i] = i < nbegin ? begin[i] : 0;
    sv[i] = i < nstride ? stride[i] : 1;
  }
  for (int i = 0; i < ndim; ++i) {
    const int64_t lo = sv[i] < 0 ? -1 : 0;
    const int64_t hi = sv[i] < 0 ? xshape[i] - 1 : xshape[i];
    int64_t b = bv[i] < 0 ? bv[i] + xshape[i] : bv[i];
    if (b < lo) b = lo;
    if (b > hi) b = hi;
    bv[i] = b;
  }
  const int64_t size = prod(yshape, ndim);
  for (int64_t i = 0; i < size; ++i) {
    int64_t t = i, src = 0, mul = 1;
    for (int j = ndim - 1; j >= 0; --j) {
      const int64_t col = t % yshape[j];
      t /= yshape[j];
      src += (bv[j] + col * sv[j]) * mul;
      mul *= xshape[j];
    }
    y[i] = x[src];
  }
  return 0;
}

int cvmo_slice_like(const int32_t* x, const int64_t* xshape, int ndim,
                    int32_t* y, const int64_t* yshape) {
  const int64_t size = prod(yshape, ndim);
  for (int64_t i = 0; i < size; ++i) {
    int64_t t = i, src = 0, mul = 1;
    for (int j = ndim - 1; j >= 0; --j) {
      src += (t % yshape[j]) * mul;
      t /= yshape[j];
      mul *= xshape[j];
    }
    y[i] = x[src];
  }
  return 0;
}

int cvmo_take(const int32_t* x, const int64_t* xshape, int xndim,
              const int32_t* indices, const int64_t* ishape, int indim,
              int32_t* y, const int64_t* yshape, int yndim, int has_axis, int axis) {
  const int64_t ysize = prod(yshape, yndim);
  if (!has_axis) {
    const int64_t xs = prod(xshape, xndim);
    for (int64_t i = 0; i < ysize; ++i) {
      int64_t j = indices[i] < 0 ? 0 : indices[i];
      if (j > xs - 1) j = xs - 1;
      y[i] = x[j];
    }
    return 0;
  }
  if (axis < 0) axis += xndim;
  if (axis < 0 || axis >= xndim || xndim > MAXD || indim > MAXD) return 1;
  int64_t xs[MAXD], is[MAXD];
  xs[xndim - 1] = 1;
  for (int i = xndim - 2; i >= 0; --i) xs[i] = xs[i + 1] * xshape[i + 1];
  is[indim - 1] = 1;
  for (int i = indim - 2; i >= 0; --i) is[i] = is[i + 1] * ishape[i + 1];
  for (int64_t i = 0; i < ysize; ++i) {
    int64_t t = i, xi = 0, ii = 0;
    for (int j = yndim - 1; j >= 0; --j) {
      const int64_t col = t % yshape[j];
      t /= yshape[j];
      if (axis <= j && j < axis + indim) ii += col * is[j - axis];
      else xi += col * xs[j < axis ? j : j - indim + 1];
      if (j == axis) {
        /* the index tensor position is complete once the walk reaches `axis` */
        int32_t v = indices[ii] < 0 ? 0 : indices[ii];
        const int32_t lim = (int32_t)xshape[axis] - 1;
        if (v > lim) v = lim;
        xi += (int64_t)v * xs[axis];
      }
    }
    y[i] = x[xi];
  }
  return 0;
}

int cvmo_repeat(const int32_t* x, const int64_t* xshape, int32_t* y, const int64_t* yshape,
                int ndim, int axis, int repeats) {
  if (axis < 0) axis += ndim;
  if (axis < 0 || axis >= ndim || repeats < 1) return 1;
  const int64_t size = prod(yshape, ndim);
  for (int64_t i = 0; i < size; ++i) {
    int64_t t = i, src = 0, mul = 1;
    for (int j = ndim - 1; j >= 0; --j) {
      int64_t col = t % yshape[j];
      t /= yshape[j];
      if (j == axis) col /= repeats;
      src += col * mul;
      mul *= xshape[j];
    }
    y[i] = x[src];
  }
  return 0;
}

int cvmo_tile(const int32_t* x, const int64_t* xshape, int xndim,
              int32_t* y, const int64_t* yshape, int yndim) {
  if (yndim < xndim) return 1;
  const int lead = yndim - xndim;
  const int64_t inner = prod(yshape + lead, xndim), outer = prod(yshape, lead);
  for (int64_t i = 0; i < inner; ++i) {
    int64_t t = i, src = 0, mul = 1;
    for (int j = xndim - 1; j >= 0; --j) {
      const int64_t col = (t % yshape[j + lead]) % xshape[j];
      t /= yshape[j + lead];
      src += col * mul;
      mul *= xshape[j];
    }
    y[i] = x[src];
  }
  for (int64_t o = 1; o < outer; ++o) memcpy(y + o * inner, y, (size_t)inner * 4);
  return 0;
}

int cvmo_upsampling(const int32_t* x, int32_t* y, int n, int c, int h, int w, int scale) {
  if (scale < 1) return 1;
  const int oh = h * scale, ow = w * scale;
  for (int64_t nc = 0; nc < (int64_t)n * c; ++nc)
    for (int p = 0; p < oh; ++p)
      for (int q = 0; q < ow; ++q)
        y[(nc * oh + p) * ow + q] = x[(nc * h + p / scale) * w + q / scale];
  return 0;
}

/* ops.cc:1061-1073.  With a 1-D condition the reference copies `size` BYTES per
 * row (not size*4), leaving the rest of each output row untouched; that is
 * restated literally. */
int cvmo_where(const int32_t* cond, const int32_t* x, const int32_t* y, int32_t* out,
               const int64_t* oshape, int ndim, int same_shape) {
  if (same_shape) {
    const int64_t size = prod(oshape, ndim);
    for (int64_t i = 0; i < size; ++i) out[i] = cond[i] == 0 ? y[i] : x[i];
  } else {
    const int64_t row = prod(oshape + 1, ndim - 1);
    for (int64_t i = 0; i < oshape[0]; ++i)
      memcpy(out + i * row, (cond[i] == 0 ? y : x) + i * row, (size_t)row);
  }
  return 0;
}

/* ---------------------------------------------------------------- detection */
int cvmo_get_valid_counts(const int32_t* x, int32_t* valid_count, int32_t* y,
                          int batches, int n, int k, int32_t score_threshold) {
  if (k < 2) return 1;
  for (int b = 0; b < batches; ++b) {
    const int32_t* in = x + (int64_t)b * n * k;
    int32_t* out = y + (int64_t)b * n * k;
    int32_t cnt = 0;
    for (int j = 0; j < n; ++j)
      if (in[(int64_t)j * k + 1] > score_threshold) {
        memcpy(out + (int64_t)cnt * k, in + (int64_t)j * k, (size_t)k * 4);
        ++cnt;
      }
    valid_count[b] = cnt;
    for (int64_t i = (int64_t)cnt * k; i < (int64_t)n * k; ++i) out[i] = -1;
  }
  return 0;
}

/* nms.cc:4-40, corner format: 100 * overlap / union, all in int64, 0 when degenerate. */
int64_t cvmo_iou(const int32_t* r1, const int32_t* r2) {
  const int64_t a1 = (int64_t)wsub(r1[2], r1[0]) * wsub(r1[3], r1[1]);
  const int64_t a2 = (int64_t)wsub(r2[2], r2[0]) * wsub(r2[3], r2[1]);
  const int64_t sum_area = (int64_t)((uint64_t)a1 + (uint64_t)a2);
  if (sum_area <= 0) return 0;
  const int32_t xr = r1[2] < r2[2] ? r1[2] : r2[2], xl = r1[0] > r2[0] ? r1[0] : r2[0];
  const int32_t yb = r1[3] < r2[3] ? r1[3] : r2[3], yt = r1[1] > r2[1] ? r1[1] : r2[1];
  int32_t w = wsub(xr, xl), h = wsub(yb, yt);
  if (w < 0) w = 0;
  if (h < 0) h = 0;
  int64_t overlap = (int64_t)h * w;
  int64_t uni = sum_area - overlap;
  if (uni <= 0) return 0;
  if (INT64_MAX / 100 < overlap) uni /= 100; else overlap *= 100;
  return overlap / uni;
}

typedef struct { int32_t score; int32_t idx; } srow_t;
static int srow_cmp(const void* a, const void* b) {
  const srow_t* p = (const srow_t*)a; const srow_t* q = (const srow_t*)b;
  if (p->score != q->score) return p->score > q->score ? -1 : 1;  /* score descending */
  return p->idx < q->idx ? -1 : (p->idx > q->idx);                /* stable: index ascending */
}

int cvmo_non_max_suppression(int32_t* x, const int32_t* valid_count, int32_t* y,
                             int batches, int n, int k, int max_output_size,
                             int iou_threshold, int topk, int coord_start,
                             int score_index, int id_index, int force_suppress) {
  if (iou_threshold <= 0) return 1; /* rejected by NMSShape (src/top/nn/nms.cc:50) */
  for (int b = 0; b < batches; ++b) {
    int32_t* xb = x + (int64_t)b * n * k;
    int32_t* yb = y + (int64_t)b * n * k;
    int vc = valid_count[b];
    if (vc > n) vc = n;
    if (vc <= 0) {
      /* nms.cc:76-79: fills this batch and returns from the whole call */
      for (int64_t i = 0; i < (int64_t)n * k; ++i) yb[i] = -1;
      return 0;
    }
    srow_t* order = (srow_t*)malloc(sizeof(srow_t) * (size_t)vc);
    unsigned char* removed = (unsigned char*)calloc((size_t)vc, 1);
    if (!order || !removed) { free(order); free(removed); return 2; }
    for (int i = 0; i < vc; ++i) { order[i].score = xb[(int64_t)i * k + score_index]; order[i].idx = i; }
    qsort(order, (size_t)vc, sizeof(srow_t), srow_cmp);
    if (topk > 0 && topk < vc)
      for (int i = topk; i < vc; ++i)
        for (int c = 0; c < k; ++c) xb[(int64_t)order[i].idx * k + c] = -1;
    const int keep = (topk >= 0 && topk < vc) ? topk : vc;
    int yi = 0;
    for (int i = 0; i < keep; ++i) {
      const int32_t* r1 = xb + (int64_t)order[i].idx * k;
      if (removed[i]) continue; /* a removed row neither emits nor suppresses */
      if (r1[0] >= 0) { memcpy(yb + (int64_t)yi * k, r1, (size_t)k * 4); ++yi; }
      for (int j = i + 1; j < keep; ++j) {
        const int32_t* r2 = xb + (int64_t)order[j].idx * k;
        if (r2[0] < 0) break; /* nms.cc:112: the scan stops at the first negative id */
        if (force_suppress || id_index < 0 || r1[id_index] == r2[id_index])
          if (cvmo_iou(r1 + coord_start, r2 + coord_start) >= iou_threshold) removed[j] = 1;
      }
    }
    for (int64_t i = (int64_t)yi * k; i < (int64_t)n * k; ++i) yb[i] = -1;
    if (max_output_size > 0) {
      int j = 0;
      for (int i = 0; i < vc; ++i)
        if (yb[(int64_t)i * k] >= 0) {
          if (j == max_output_size) for (int c = 0; c < k; ++c) yb[(int64_t)i * k + c] = -1;
          else ++j;
        }
    }
    free(order);
    free(removed);
  }
  return 0;
}
