// Entry points of the fused int8 path: int8 activations (layout: conv_mfma.h) between layers,
// requantisation chains folded into the producing kernel.  The arithmetic of
// every stage is the operator's own (int32, wrapping), so results equal the
// node-by-node execution bit for bit.
#include "conv_mfma.h"

namespace cvmhip {

__device__ __forceinline__ uint32_t pack4(int32_t a, int32_t b, int32_t c, int32_t d) {
  return (uint32_t)(uint8_t)(int8_t)a | ((uint32_t)(uint8_t)(int8_t)b << 8) | ((uint32_t)(uint8_t)(int8_t)c << 16) |
         ((uint32_t)(uint8_t)(int8_t)d << 24);
}
__device__ __forceinline__ int32_t byte_of(uint32_t w, int e) { return (int32_t)(int8_t)(w >> (8 * e)); }

// All kernels below run one thread per dword (4 channels of one pixel) of the
// int8 result, in memory order, whatever the layout (conv_mfma.h: act_decode).

// out = chain(a + b)
__global__ void __launch_bounds__(256)
k_add_i8(const uint32_t* __restrict__ a, const uint32_t* __restrict__ b, void* __restrict__ out, int out_is_i8,
         int64_t total, int64_t npix, int c, int cp, int hw, DevChain chain) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const uint32_t u = a[i], v = b[i];
    int32_t r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = apply_chain(chain, byte_of(u, e) + byte_of(v, e));
    if (out_is_i8) {
      reinterpret_cast<uint32_t*>(out)[i] = pack4(r[0], r[1], r[2], r[3]);
    } else {
      int64_t pixel;
      int c0;
      act_decode(i, cp, &pixel, &c0);
      if (pixel >= npix) continue;
      const int64_t n = pixel / hw;
      const int pix = (int)(pixel - n * hw);
      int32_t* y = reinterpret_cast<int32_t*>(out) + (n * c) * hw + pix;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c0 + e < c) y[(int64_t)(c0 + e) * hw] = r[e];
    }
  }
}

__global__ void __launch_bounds__(256)
k_max_pool_i8(const uint32_t* __restrict__ x, uint32_t* __restrict__ y, int64_t total, int64_t npix_out, int cp, int h, int w,
              int oh, int ow, int kh, int kw, int sh, int sw, int ph, int pw) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    int64_t t;
    int c0;
    act_decode(i, cp, &t, &c0);
    if (t >= npix_out) continue;
    const int q = (int)(t % ow);
    t /= ow;
    const int p = (int)(t % oh);
    const int64_t n = t / oh;
    int32_t m[4] = {-128, -128, -128, -128};
    for (int r = 0; r < kh; ++r) {
      const int ih = p * sh + r - ph;
      if (ih < 0 || ih >= h) continue;
      for (int s = 0; s < kw; ++s) {
        const int iw = q * sw + s - pw;
        if (iw < 0 || iw >= w) continue;
        const uint32_t v = x[act_offset((n * h + ih) * w + iw, c0, cp) >> 2];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int32_t b = byte_of(v, e);
          m[e] = b > m[e] ? b : m[e];
        }
      }
    }
    y[i] = pack4(m[0], m[1], m[2], m[3]);
  }
}

// max_pool2d for Cp >= 16: one thread per 16 channels of one output pixel (16-byte loads and stores)
// The common windows (KH, KW > 0: 3x3 and 2x2): every tap of a granule requested before the first is used, G granules
// per thread in flight (see max_pool_request); KH = 0: any window, tap by tap.
template <int KH, int KW>
__global__ void __launch_bounds__(256)
k_max_pool_i8x16(const int8_t* __restrict__ x, int8_t* __restrict__ y, int64_t total, int64_t npix_out, int cp, int h,
                 int w, int oh, int ow, int kh, int kw, int sh, int sw, int ph, int pw, FastDiv div_ow, FastDiv div_oh) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  if constexpr (KH > 0) {
    constexpr int G = 2;
    auto load = [&](int64_t off) __attribute__((always_inline)) { return *reinterpret_cast<const int4*>(x + off); };
    for (int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i0 < total; i0 += G * stride) {
      int4 v[G][KH * KW];
      bool ok[G];
#pragma unroll
      for (int k = 0; k < G; ++k) {
        const int64_t i = i0 + k * stride;
        int64_t t;
        int c0;
        act_decode((i < total ? i : i0) * 4, cp, &t, &c0);
        ok[k] = i < total && t < npix_out;
        if (t >= npix_out) t = npix_out - 1;
        const unsigned row = fastdiv((unsigned)t, div_ow);          // npix_out < 2^31 (checked by the host)
        const int q = (int)((unsigned)t - row * (unsigned)ow);
        const unsigned n = fastdiv(row, div_oh);
        const int p = (int)(row - n * (unsigned)oh);
        max_pool_request<KH, KW>(v[k], load, (int)n, p, q, c0, cp, h, w, sh, sw, ph, pw);
      }
#pragma unroll
      for (int k = 0; k < G; ++k)
        if (ok[k]) *reinterpret_cast<int4*>(y + (i0 + k * stride) * 16) = max_pool_reduce<KH * KW>(v[k]);
    }
    return;
  }
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    int64_t t;
    int c0;
    act_decode(i * 4, cp, &t, &c0);
    if (t >= npix_out) continue;
    const int q = (int)(t % ow);
    t /= ow;
    const int p = (int)(t % oh);
    const int64_t n = t / oh;
    int32_t m[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) m[e] = -128;
    for (int r = 0; r < kh; ++r) {
      const int ih = p * sh + r - ph;
      if (ih < 0 || ih >= h) continue;
      for (int s = 0; s < kw; ++s) {
        const int iw = q * sw + s - pw;
        if (iw < 0 || iw >= w) continue;
        const int4 v = *reinterpret_cast<const int4*>(x + act_offset((n * h + ih) * w + iw, c0, cp));
        const uint32_t d[4] = {(uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w};
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int32_t b = byte_of(d[e >> 2], e & 3);
          m[e] = b > m[e] ? b : m[e];
        }
      }
    }
    *reinterpret_cast<int4*>(y + i * 16) = make_int4(pack4(m[0], m[1], m[2], m[3]), pack4(m[4], m[5], m[6], m[7]),
                                                     pack4(m[8], m[9], m[10], m[11]), pack4(m[12], m[13], m[14], m[15]));
  }
}

// out[n][c] = chain(sum_hw x[n][hw][c]); the result is a tensor of n "pixels"
// Sixteen consecutive lanes share one output dword (4 channels of one image): each sums every sixteenth pixel,
// four requests at a time (a lane's requests would otherwise wait for one another: the layer is a handful of
// round trips to memory and nothing else), and a butterfly over the 16 lanes adds the parts.
constexpr int SUM_LANES = 16;
__global__ void __launch_bounds__(256)
k_sum_hw_i8(const uint32_t* __restrict__ x, void* __restrict__ out, int out_is_i8, int64_t total, int nimg, int c, int cp,
            int hw, DevChain chain) {
  const int64_t stride = ((int64_t)gridDim.x * blockDim.x) / SUM_LANES;
  const int part = threadIdx.x & (SUM_LANES - 1);
  // all lanes of a group run the same number of iterations (total is rounded up by the launch)
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / SUM_LANES; i < total; i += stride) {
    int64_t n;
    int c0;
    act_decode(i, cp, &n, &c0);
    int32_t acc[4] = {0, 0, 0, 0};
    if (n < nimg) {
      for (int t = part; t < hw; t += 4 * SUM_LANES) {
        uint32_t v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int tt = t + SUM_LANES * k;
          v[k] = x[act_offset(n * hw + (tt < hw ? tt : t), c0, cp) >> 2];
          if (tt >= hw) v[k] = 0;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] += byte_of(v[k], e);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[e] += __shfl_xor(acc[e], 1, 64);
      acc[e] += __shfl_xor(acc[e], 2, 64);
      acc[e] += __shfl_xor(acc[e], 4, 64);
      acc[e] += __shfl_xor(acc[e], 8, 64);
    }
    if (part != 0 || n >= nimg) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = apply_chain(chain, acc[e]);
    if (out_is_i8) {
      reinterpret_cast<uint32_t*>(out)[i] = pack4(acc[0], acc[1], acc[2], acc[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c0 + e < c) reinterpret_cast<int32_t*>(out)[n * c + c0 + e] = acc[e];
    }
  }
}

// depthwise convolution; filter is [tap][cp] int8
__global__ void __launch_bounds__(256)
k_depthwise_i8(const uint32_t* __restrict__ x, const uint32_t* __restrict__ wp, const int32_t* __restrict__ bias,
               void* __restrict__ out, int out_is_i8, int64_t total, int64_t npix_out, int c, int cp, int h, int w, int oh,
               int ow, int kh, int kw, int sh, int sw, int ph, int pw, int dh, int dw, DevChain chain) {
  const int c4n = cp >> 2;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    int64_t t;
    int c0;
    act_decode(i, cp, &t, &c0);
    if (t >= npix_out) continue;
    const int q = (int)(t % ow);
    t /= ow;
    const int p = (int)(t % oh);
    const int64_t n = t / oh;
    int32_t acc[4] = {0, 0, 0, 0};
    for (int r = 0; r < kh; ++r) {
      const int ih = p * sh + r * dh - ph;
      if (ih < 0 || ih >= h) continue;
      for (int s = 0; s < kw; ++s) {
        const int iw = q * sw + s * dw - pw;
        if (iw < 0 || iw >= w) continue;
        const uint32_t v = x[act_offset((n * h + ih) * w + iw, c0, cp) >> 2];
        const uint32_t f = wp[(r * kw + s) * c4n + (c0 >> 2)];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += byte_of(v, e) * byte_of(f, e);
      }
    }
    int32_t rr[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ch = c0 + e;
      rr[e] = ch < c ? apply_chain(chain, wadd(acc[e], bias ? bias[ch] : 0)) : 0;
    }
    if (out_is_i8) {
      reinterpret_cast<uint32_t*>(out)[i] = pack4(rr[0], rr[1], rr[2], rr[3]);
    } else {
      int32_t* y = reinterpret_cast<int32_t*>(out) + ((n * c) * oh + p) * ow + q;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c0 + e < c) y[(int64_t)(c0 + e) * oh * ow] = rr[e];
    }
  }
}

// int32 [c][1][kh][kw] -> int8 [tap][cp]
__global__ void __launch_bounds__(256)
k_pack_depthwise(const int32_t* __restrict__ w, int8_t* __restrict__ wp, int64_t total, int c, int cp, int taps) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int ch = (int)(i % cp);
    const int tap = (int)(i / cp);
    wp[i] = ch < c ? (int8_t)w[(int64_t)ch * taps + tap] : 0;
  }
}

// int8 act tensor of n images x hw pixels x cp channels (cp % 32 == 0) -> int8 act tensor of n "pixels" (one per image)
// x hw * cp channels, channel p * cp + c of image i = channel c of the image's pixel p.  One 16-byte granule (16
// channels of one pixel) per thread; rows n .. 31 of the destination's pixel block are not written.
__global__ void __launch_bounds__(256)
k_flatten_act(const int8_t* __restrict__ xp, int8_t* __restrict__ yp, unsigned granules, unsigned n, unsigned hw, unsigned cp) {
  const unsigned gpp = cp >> 4;   // granules per pixel
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;   // (32-bit arithmetic throughout: the host bounds the sizes)
  if (i >= granules) return;
  const unsigned kg = i / n;             // granule of the flattened channel axis
  const unsigned img = i - kg * n;       // consecutive threads: the rows of one destination block half
  const unsigned p = kg / gpp;
  const unsigned c = (kg - p * gpp) * 16u;
  const int4 v = *reinterpret_cast<const int4*>(xp + act_offset((int64_t)(img * hw + p), (int)c, (int)cp));
  *reinterpret_cast<int4*>(yp + act_offset((int64_t)img, (int)(kg * 16u), (int)(hw * cp))) = v;
}

}  // namespace cvmhip

using namespace cvmhip;

extern "C" {

int cvmhip_pad_channels(int channels) { return pad_channels(channels); }

int cvmhip_flatten_act_i8(const void* xp, void* yp, int n, int c, int hw, void* stream) {
  if (!xp || !yp || n < 1 || c < 32 || (c & 31) || hw < 1 || (int64_t)hw * c > (1 << 28) || (int64_t)n * hw * c > (1ll << 31) - 4096 ||
      (((uintptr_t)xp | (uintptr_t)yp) & 15))
    return arg_error("flatten_act_i8 (channels a multiple of 32, 16-byte aligned tensors, less than 2 GiB)");
  hipStream_t s = as_stream(stream);
  const unsigned granules = (unsigned)((int64_t)n * hw * (c >> 4));
  KernelTimer timer("k_flatten_act", 2.0 * (double)granules * 16.0, s);   // bytes in + out
  k_flatten_act<<<(granules + 255) / 256, 256, 0, s>>>(reinterpret_cast<const int8_t*>(xp), reinterpret_cast<int8_t*>(yp), granules,
                                                      (unsigned)n, (unsigned)hw, (unsigned)c);
  return check_launch("flatten_act_i8");
}

int cvmhip_pack_nhwc_i8(const int32_t* x, void* xp, int n, int c, int hw, void* stream) {
  if (!x || !xp || n < 1 || c < 1 || hw < 1 || ((uintptr_t)xp & 3)) return arg_error("pack_nhwc_i8");
  return pack_activations(x, reinterpret_cast<int8_t*>(xp), n, c, hw, as_stream(stream));
}

int cvmhip_unpack_nhwc_i8(const void* xp, int32_t* x, int n, int c, int hw, void* stream) {
  if (!x || !xp || n < 1 || c < 1 || hw < 1) return arg_error("unpack_nhwc_i8");
  return unpack_activations(reinterpret_cast<const int8_t*>(xp), x, n, c, hw, as_stream(stream));
}

static int conv2d_i8_any(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                         const void* residual, const cvmhip_chain* chain2, void* out, int out_is_i8, int64_t nhwc_image_stride,
                         int n, int ic, int h, int wd, int oc, int kh, int kw,
                         int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream,
                         void* ws = nullptr, size_t ws_bytes = 0, size_t* ws_query = nullptr, void* seq_table = nullptr,
                         int seq_index = 0, int pool = 0, int* pool_query = nullptr, void* group_table = nullptr,
                         int group_index = 0, int group_first = 0, int* group_blocks = nullptr) {
  if (!xp || !wp || !out) return arg_error("conv2d_i8 null tensor");
  if (n < 1 || ic < 1 || h < 1 || wd < 1 || oc < 1 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
      pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1)
    return arg_error("conv2d_i8 attributes");
  if (h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1)
    return arg_error("conv2d_i8 kernel exceeds input");
  ConvGeom g = {};
  g.N = n; g.H = h; g.W = wd; g.Cp = pad_channels(ic); g.C = ic;
  g.OC = oc;
  g.OH = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  g.OW = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = pad_h; g.PW = pad_w; g.DH = dil_h; g.DW = dil_w;
  Epilogue ep = {};
  ep.bias = bias;
  if (!make_chain(chain, &ep.chain) || !make_chain(chain2, &ep.chain2)) return arg_error("conv2d_i8 chain");
  ep.residual = reinterpret_cast<const int8_t*>(residual);
  ep.out_mode = out_is_i8 ? OUT_I8_ACT : OUT_I32_NCHW;
  ep.out_cp = pad_channels(oc);
  if (nhwc_image_stride >= 0) {
    if (out_is_i8 || nhwc_image_stride < (int64_t)g.OH * g.OW * oc) return arg_error("conv2d_i8_nhwc image stride");
    ep.o32_img = nhwc_image_stride;
    ep.o32_ch = 1;
    ep.o32_px = oc;
  }
  ep.pool = pool;
  if (pool_query) {   // eligibility question only
    *pool_query = conv_pool_eligible(g) ? 1 : 0;
    return CVMHIP_OK;
  }
  if (ws_query) {   // size question only
    *ws_query = nhwc_image_stride >= 0 ? 0 : conv_slices_workspace_bytes(g, ep);
    return CVMHIP_OK;
  }
  if (group_table)   // describe the launch as one entry of a launch of independent convolutions
    return conv_group_layer(group_table, group_index, group_first, reinterpret_cast<const int8_t*>(xp), reinterpret_cast<const int8_t*>(wp),
                            out, g, ep, group_blocks);
  if (seq_table)   // describe the launch as one layer of a layer-sequence launch instead of issuing it
    return conv_seq_layer(seq_table, seq_index, reinterpret_cast<const int8_t*>(xp), reinterpret_cast<const int8_t*>(wp), out, g, ep);
  if (nhwc_image_stride >= 0) ws = nullptr;
  return conv_igemm_ws(reinterpret_cast<const int8_t*>(xp), reinterpret_cast<const int8_t*>(wp), out, g, ep, ws, ws_bytes,
                       as_stream(stream));
}

size_t cvmhip_conv2d_i8_workspace_bytes(int has_residual, int n, int ic, int h, int wd, int oc, int kh, int kw,
                                        int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w) {
  size_t bytes = 0;
  const int dummy = 0;
  const int rc = conv2d_i8_any(&dummy, &dummy, nullptr, nullptr, has_residual ? &dummy : nullptr, nullptr, const_cast<int*>(&dummy), 1, -1,
                               n, ic, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, nullptr, nullptr, 0, &bytes);
  return rc == CVMHIP_OK ? bytes : 0;
}

int cvmhip_conv2d_i8_ws(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                        const void* residual, const cvmhip_chain* chain2, void* out, int out_is_i8,
                        int n, int ic, int h, int wd, int oc, int kh, int kw,
                        int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return conv2d_i8_any(xp, wp, bias, chain, residual, chain2, out, out_is_i8, -1, n, ic, h, wd, oc, kh, kw, stride_h, stride_w,
                       pad_h, pad_w, dil_h, dil_w, stream, workspace, workspace_bytes);
}

int cvmhip_conv2d_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                     const void* residual, const cvmhip_chain* chain2, void* out, int out_is_i8,
                     int n, int ic, int h, int wd, int oc, int kh, int kw,
                     int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  return conv2d_i8_any(xp, wp, bias, chain, residual, chain2, out, out_is_i8, -1, n, ic, h, wd, oc, kh, kw, stride_h, stride_w,
                       pad_h, pad_w, dil_h, dil_w, stream);
}

int cvmhip_conv2d_pool2_i8_eligible(int n, int ic, int h, int wd, int oc, int kh, int kw,
                                    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w) {
  int yes = 0;
  const int dummy = 0;
  const int rc = conv2d_i8_any(&dummy, &dummy, nullptr, nullptr, nullptr, nullptr, const_cast<int*>(&dummy), 1, -1, n, ic, h, wd, oc, kh,
                               kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, nullptr, nullptr, 0, nullptr, nullptr, 0, 1, &yes);
  return rc == CVMHIP_OK ? yes : 0;
}

int cvmhip_conv2d_pool2_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain, void* out,
                           int n, int ic, int h, int wd, int oc, int kh, int kw,
                           int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  return conv2d_i8_any(xp, wp, bias, chain, nullptr, nullptr, out, 1, -1, n, ic, h, wd, oc, kh, kw, stride_h, stride_w,
                       pad_h, pad_w, dil_h, dil_w, stream, nullptr, 0, nullptr, nullptr, 0, 1);
}

size_t cvmhip_conv_seq_layer_bytes(void) { return conv_seq_layer_bytes(); }
size_t cvmhip_conv_seq_sync_bytes(void) { return conv_seq_sync_bytes(); }
int cvmhip_conv_seq_shares(void) { return conv_seq_shares(); }

int cvmhip_conv_seq_layer(void* table, int index, const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          const void* residual, const cvmhip_chain* chain2, void* out,
                          int n, int ic, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w) {
  if (!table || index < 0) return arg_error("conv_seq_layer table");
  return conv2d_i8_any(xp, wp, bias, chain, residual, chain2, out, 1, -1, n, ic, h, wd, oc, kh, kw, stride_h, stride_w,
                       pad_h, pad_w, dil_h, dil_w, nullptr, nullptr, 0, nullptr, table, index);
}

int cvmhip_conv_seq_layer_config(const void* table, int index) {
  if (!table || index < 0) return -1;
  return conv_seq_layer_config(table, index);
}

int cvmhip_conv_seq_layer_chain(const void* table, int index) {
  if (!table || index < 0) return 0;
  return conv_seq_layer_chain(table, index);
}

int cvmhip_conv_seq_link(void* table, int count) {
  if (!table || count < 1) return 0;
  return conv_seq_link(table, count);
}

int cvmhip_conv_seq_launch(const void* dev_table, int nlayers, void* sync, double ops, double bytes, void* stream) {
  return conv_seq_launch(dev_table, nlayers, sync, ops, bytes, as_stream(stream));
}

int cvmhip_conv2d_i8_nhwc(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          int32_t* out, int64_t image_stride, int n, int ic, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  if (image_stride < 0) return arg_error("conv2d_i8_nhwc image stride");
  return conv2d_i8_any(xp, wp, bias, chain, nullptr, nullptr, out, 0, image_stride, n, ic, h, wd, oc, kh, kw, stride_h, stride_w,
                       pad_h, pad_w, dil_h, dil_w, stream);
}

size_t cvmhip_packed_weight_pair_bytes(int oc_a, int oc_b, int ic, int kh, int kw) {
  if (oc_a < 1 || oc_b < 1 || ic < 1 || kh < 1 || kw < 1) return 0;
  return packed_weight_pair_bytes(oc_a, oc_b, ic, kh, kw);
}

int cvmhip_pack_weights_pair(const int32_t* w_a, int oc_a, const int32_t* w_b, int oc_b, void* wp, int ic, int kh, int kw, void* stream) {
  if (!w_a || !w_b || !wp || ((uintptr_t)wp & 15) || oc_a < 1 || oc_b < 1 || ic < 1 || kh < 1 || kw < 1) return arg_error("pack_weights_pair");
  return pack_weights_pair(w_a, oc_a, w_b, oc_b, reinterpret_cast<int8_t*>(wp), ic, kh, kw, as_stream(stream));
}

// One or two detection heads over one tensor: launched, or recorded as entry `group_index` of a table of independent
// convolutions (group_table != NULL; its workgroups begin at first_block, *blocks receives their number).
static int heads_any(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                     int32_t* out_a, int64_t image_stride_a, int oc_a, int32_t* out_b, int64_t image_stride_b, int oc_b,
                     int n, int ic, int h, int wd, int kh, int kw,
                     int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream,
                     void* group_table, int group_index, int first_block, int* blocks) {
  if (!xp || !wp || !out_a) return arg_error("detection heads: null tensor");
  if (n < 1 || ic < 1 || h < 1 || wd < 1 || oc_a < 1 || (out_b && oc_b < 1) || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
      pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1)
    return arg_error("detection heads: attributes");
  if (h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1)
    return arg_error("detection heads: kernel exceeds input");
  const int split = out_b ? (oc_a + 31) / 32 * 32 : 0;
  ConvGeom g = {};
  g.N = n; g.H = h; g.W = wd; g.Cp = pad_channels(ic); g.C = ic;
  g.OC = out_b ? split + oc_b : oc_a;
  g.OH = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  g.OW = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = pad_h; g.PW = pad_w; g.DH = dil_h; g.DW = dil_w;
  if (image_stride_a < (int64_t)g.OH * g.OW * oc_a || (out_b && image_stride_b < (int64_t)g.OH * g.OW * oc_b))
    return arg_error("detection heads: image stride");
  Epilogue ep = {};
  ep.bias = bias;
  if (!make_chain(chain, &ep.chain) || !make_chain(nullptr, &ep.chain2)) return arg_error("detection heads: chain");
  ep.out_mode = OUT_I32_NCHW;
  ep.out_cp = pad_channels(g.OC);
  ep.o32_img = image_stride_a; ep.o32_ch = 1; ep.o32_px = oc_a;
  if (out_b) {
    ep.split = split; ep.oc_a = oc_a; ep.oc_b = oc_b;
    ep.o32_img_b = image_stride_b; ep.o32_ch_b = 1; ep.o32_px_b = oc_b;
    ep.out_b = out_b;
  }
  if (group_table)
    return conv_group_layer(group_table, group_index, first_block, reinterpret_cast<const int8_t*>(xp),
                            reinterpret_cast<const int8_t*>(wp), out_a, g, ep, blocks);
  return conv_igemm(reinterpret_cast<const int8_t*>(xp), reinterpret_cast<const int8_t*>(wp), out_a, g, ep, as_stream(stream));
}

int cvmhip_conv2d_i8_nhwc_pair(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                               int32_t* out_a, int64_t image_stride_a, int oc_a, int32_t* out_b, int64_t image_stride_b, int oc_b,
                               int n, int ic, int h, int wd, int kh, int kw,
                               int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  if (!out_b) return arg_error("conv2d_i8_nhwc_pair null tensor");
  return heads_any(xp, wp, bias, chain, out_a, image_stride_a, oc_a, out_b, image_stride_b, oc_b, n, ic, h, wd, kh, kw, stride_h,
                   stride_w, pad_h, pad_w, dil_h, dil_w, stream, nullptr, 0, 0, nullptr);
}

size_t cvmhip_conv_group_layer_bytes(void) { return conv_seq_layer_bytes(); }

int cvmhip_conv_group_heads(void* table, int index, int first_block, int* blocks, const void* xp, const void* wp, const int32_t* bias,
                            const cvmhip_chain* chain, int32_t* out_a, int64_t image_stride_a, int oc_a, int32_t* out_b,
                            int64_t image_stride_b, int oc_b, int n, int ic, int h, int wd, int kh, int kw,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w) {
  if (!table || index < 0 || !blocks) return arg_error("conv_group_heads table");
  return heads_any(xp, wp, bias, chain, out_a, image_stride_a, oc_a, out_b, image_stride_b, oc_b, n, ic, h, wd, kh, kw, stride_h,
                   stride_w, pad_h, pad_w, dil_h, dil_w, nullptr, table, index, first_block, blocks);
}

int cvmhip_conv_group_launch(const void* dev_table, int nlayers, int total_blocks, double ops, double bytes, void* stream) {
  return conv_group_launch(dev_table, nlayers, total_blocks, 0, ops, bytes, as_stream(stream));
}

int cvmhip_conv_group_conv_i8(void* table, int index, int first_block, int* blocks, const void* xp, const void* wp, const int32_t* bias,
                              const cvmhip_chain* chain, const void* residual, const cvmhip_chain* chain2, void* out,
                              int n, int ic, int h, int wd, int oc, int kh, int kw,
                              int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w) {
  if (!table || index < 0 || !blocks) return arg_error("conv_group_conv_i8 table");
  return conv2d_i8_any(xp, wp, bias, chain, residual, chain2, out, 1, -1, n, ic, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w,
                       dil_h, dil_w, nullptr, nullptr, 0, nullptr, nullptr, 0, 0, nullptr, table, index, first_block, blocks);
}

int cvmhip_conv_group_launch_i8(const void* dev_table, int nlayers, int total_blocks, double ops, double bytes, void* stream) {
  return conv_group_launch(dev_table, nlayers, total_blocks, 1, ops, bytes, as_stream(stream));
}

// ---- row-window convolution over at most 4 input channels (the RGB stem of a network)
int cvmhip_stem_eligible(int c, int kh, int kw, int dil_h, int dil_w) { return stem_eligible(c, kh, kw, dil_h, dil_w) ? 1 : 0; }

size_t cvmhip_stem_input_bytes(int n, int h, int w, int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w) {
  if (n < 1 || h < 1 || w < 1 || kh < 1 || kw < 1 || kw > 8 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0 ||
      h + 2 * pad_h < kh || w + 2 * pad_w < kw)
    return 0;
  return stem_geom(n, h, w, kh, kw, stride_h, stride_w, pad_h, pad_w).bytes;
}

int cvmhip_pack_stem_input(const int32_t* x, void* xs, int n, int c, int h, int w, int kh, int kw,
                           int stride_h, int stride_w, int pad_h, int pad_w, void* stream) {
  if (!x || !xs || ((uintptr_t)xs & 15) || !stem_eligible(c, kh, kw, 1, 1) ||
      cvmhip_stem_input_bytes(n, h, w, kh, kw, stride_h, stride_w, pad_h, pad_w) == 0)
    return arg_error("pack_stem_input");
  return pack_stem_input(x, reinterpret_cast<int8_t*>(xs), n, c, h, w, kh, kw, stride_h, stride_w, pad_h, pad_w, as_stream(stream));
}

size_t cvmhip_packed_stem_weight_bytes(int oc, int kh, int kw) {
  if (oc < 1 || kh < 1 || kw < 1 || kw > 8) return 0;
  const int rb = kw * 4 <= 16 ? 16 : 32;
  return packed_stem_weight_bytes(oc, (kh * rb + 63) / 64 * 64);
}

int cvmhip_pack_stem_weights(const int32_t* w, void* wp, int oc, int c, int kh, int kw, void* stream) {
  if (!w || !wp || oc < 1 || !stem_eligible(c, kh, kw, 1, 1)) return arg_error("pack_stem_weights");
  return pack_stem_weights(w, reinterpret_cast<int8_t*>(wp), oc, c, kh, kw, as_stream(stream));
}

int cvmhip_conv2d_stem_i8(const void* xs, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          void* out, int out_is_i8, int n, int c, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, void* stream) {
  if (!xs || !wp || !out || oc < 1 || !stem_eligible(c, kh, kw, 1, 1) ||
      cvmhip_stem_input_bytes(n, h, wd, kh, kw, stride_h, stride_w, pad_h, pad_w) == 0)
    return arg_error("conv2d_stem_i8");
  const StemGeom sg = stem_geom(n, h, wd, kh, kw, stride_h, stride_w, pad_h, pad_w);
  ConvGeom g = {};
  g.N = n; g.H = sg.hp; g.W = sg.wp; g.Cp = 4; g.C = c;
  g.OC = oc;
  g.OH = (h + 2 * pad_h - kh) / stride_h + 1;
  g.OW = (wd + 2 * pad_w - kw) / stride_w + 1;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = 0; g.PW = 0; g.DH = 1; g.DW = 1;
  g.row_bytes = sg.row_bytes;
  Epilogue ep = {};
  ep.bias = bias;
  if (!make_chain(chain, &ep.chain)) return arg_error("conv2d_stem_i8 chain");
  ep.out_mode = out_is_i8 ? OUT_I8_ACT : OUT_I32_NCHW;
  ep.out_cp = pad_channels(oc);
  return conv_igemm(reinterpret_cast<const int8_t*>(xs), reinterpret_cast<const int8_t*>(wp), out, g, ep, as_stream(stream));
}

int cvmhip_conv2d_stem_pool3_i8_eligible(int n, int c, int h, int wd, int oc, int kh, int kw, int stride_h, int stride_w,
                                         int pad_h, int pad_w, int pool_oh, int pool_ow) {
  if (n < 1 || h < 1 || wd < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0 || kh < 1 || kw < 1 ||
      cvmhip_stem_input_bytes(n, h, wd, kh, kw, stride_h, stride_w, pad_h, pad_w) == 0)
    return 0;
  return stem_pool_eligible(c, oc, kh, kw, (h + 2 * pad_h - kh) / stride_h + 1, (wd + 2 * pad_w - kw) / stride_w + 1, pool_oh, pool_ow) ? 1 : 0;
}

int cvmhip_conv2d_stem_pool3_i8(const void* xs, const void* wp, const int32_t* bias, const cvmhip_chain* chain, void* out,
                                int n, int c, int h, int wd, int oc, int kh, int kw, int stride_h, int stride_w,
                                int pad_h, int pad_w, int pool_oh, int pool_ow, void* stream) {
  if (!xs || !wp || !out || !cvmhip_conv2d_stem_pool3_i8_eligible(n, c, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, pool_oh, pool_ow))
    return arg_error("conv2d_stem_pool3_i8: not eligible");
  DevChain ch;
  if (!make_chain(chain, &ch)) return arg_error("conv2d_stem_pool3_i8 chain");
  return stem_pool(reinterpret_cast<const int8_t*>(xs), reinterpret_cast<const int8_t*>(wp), bias, ch, reinterpret_cast<int8_t*>(out),
                   n, c, h, wd, oc, kh, kw, stride_h, stride_w, pad_h, pad_w, pool_oh, pool_ow, as_stream(stream));
}

size_t cvmhip_packed_depthwise_bytes(int c, int kh, int kw) {
  return ((size_t)pad_channels(c) * kh * kw + 255) / 256 * 256;
}

int cvmhip_pack_depthwise_weights(const int32_t* w, void* wp, int c, int kh, int kw, void* stream) {
  if (!w || !wp || c < 1 || kh < 1 || kw < 1) return arg_error("pack_depthwise_weights");
  const int cp = pad_channels(c);
  const int64_t total = (int64_t)cp * kh * kw;
  k_pack_depthwise<<<grid_for(total, 256), 256, 0, as_stream(stream)>>>(w, reinterpret_cast<int8_t*>(wp), total, c, cp,
                                                                       kh * kw);
  return check_launch("pack_depthwise");
}

// ---- depthwise convolution on the matrix cores: each tile of 32 output channels is a convolution over its own
// 32 input channels with a diagonal filter matrix per tap
int cvmhip_depthwise_mfma_eligible(int c, int kh, int kw) {
  return c >= 1 && kh >= 1 && kw >= 1 && kh <= 32 && kw <= 32 && (pad_channels(c) % 32) == 0 ? 1 : 0;
}

size_t cvmhip_packed_depthwise_mfma_bytes(int c, int kh, int kw) {
  if (!cvmhip_depthwise_mfma_eligible(c, kh, kw)) return 0;
  return packed_depthwise_diag_bytes(c, kh, kw);
}

int cvmhip_pack_depthwise_weights_mfma(const int32_t* w, void* wp, int c, int kh, int kw, void* stream) {
  if (!w || !wp || ((uintptr_t)wp & 15) || !cvmhip_depthwise_mfma_eligible(c, kh, kw)) return arg_error("pack_depthwise_weights_mfma");
  return pack_depthwise_diag(w, reinterpret_cast<int8_t*>(wp), c, kh, kw, as_stream(stream));
}

int cvmhip_depthwise_conv2d_mfma_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                                    void* out, int out_is_i8, int n, int c, int h, int wd, int kh, int kw,
                                    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  if (!xp || !wp || !out) return arg_error("depthwise_conv2d_mfma_i8 null tensor");
  if (n < 1 || h < 1 || wd < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1 ||
      !cvmhip_depthwise_mfma_eligible(c, kh, kw) || h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1)
    return arg_error("depthwise_conv2d_mfma_i8 attributes");
  ConvGeom g = {};
  g.N = n; g.H = h; g.W = wd; g.Cp = pad_channels(c); g.C = c;
  g.OC = c;
  g.OH = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  g.OW = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = pad_h; g.PW = pad_w; g.DH = dil_h; g.DW = dil_w;
  g.dw = 1;
  Epilogue ep = {};
  ep.bias = bias;
  if (!make_chain(chain, &ep.chain) || !make_chain(nullptr, &ep.chain2)) return arg_error("depthwise_conv2d_mfma_i8 chain");
  ep.out_mode = out_is_i8 ? OUT_I8_ACT : OUT_I32_NCHW;
  ep.out_cp = pad_channels(c);
  return conv_igemm(reinterpret_cast<const int8_t*>(xp), reinterpret_cast<const int8_t*>(wp), out, g, ep, as_stream(stream));
}

int cvmhip_depthwise_conv2d_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                               void* out, int out_is_i8, int n, int c, int h, int wd, int kh, int kw,
                               int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream) {
  if (!xp || !wp || !out) return arg_error("depthwise_conv2d_i8 null tensor");
  if (n < 1 || c < 1 || h < 1 || wd < 1 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 || pad_h < 0 || pad_w < 0 ||
      dil_h < 1 || dil_w < 1 || h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1)
    return arg_error("depthwise_conv2d_i8 attributes");
  if (((uintptr_t)xp | (uintptr_t)wp | (uintptr_t)out) & 3) return arg_error("depthwise_conv2d_i8 alignment");
  DevChain ch;
  if (!make_chain(chain, &ch)) return arg_error("depthwise_conv2d_i8 chain");
  const int oh = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  const int ow = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  const int cp = pad_channels(c);
  const int64_t npix = (int64_t)n * oh * ow;
  const int64_t total = act_bytes(npix, cp) / 4;
  hipStream_t s = as_stream(stream);
  KernelTimer timer("k_depthwise_i8", (double)n * c * ((double)h * wd + (double)oh * ow), s);  // bytes in + out
  k_depthwise_i8<<<grid_for(total, 256, 1 << 16), 256, 0, s>>>(
      reinterpret_cast<const uint32_t*>(xp), reinterpret_cast<const uint32_t*>(wp), bias, out, out_is_i8, total, npix, c, cp,
      h, wd, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, ch);
  return check_launch("depthwise_conv2d_i8");
}

int cvmhip_add_i8(const void* a, const void* b, const cvmhip_chain* chain, void* out, int out_is_i8,
                  int n, int c, int hw, void* stream) {
  if (!a || !b || !out || n < 1 || c < 1 || hw < 1) return arg_error("add_i8");
  if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) & 3) return arg_error("add_i8 alignment");
  DevChain ch;
  if (!make_chain(chain, &ch)) return arg_error("add_i8 chain");
  const int cp = pad_channels(c);
  const int64_t npix = (int64_t)n * hw;
  const int64_t total = act_bytes(npix, cp) / 4;
  hipStream_t s = as_stream(stream);
  KernelTimer timer("k_add_i8", (double)n * c * hw * 3.0, s);
  k_add_i8<<<grid_for(total, 256), 256, 0, s>>>(reinterpret_cast<const uint32_t*>(a), reinterpret_cast<const uint32_t*>(b),
                                                out, out_is_i8, total, npix, c, cp, hw, ch);
  return check_launch("add_i8");
}

int cvmhip_max_pool2d_i8(const void* xp, void* yp, int n, int c, int h, int w, int oh, int ow,
                         int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w, void* stream) {
  if (!xp || !yp || n < 1 || c < 1 || h < 1 || w < 1 || oh < 1 || ow < 1 || kh < 1 || kw < 1 || stride_h < 1 ||
      stride_w < 1 || pad_h < 0 || pad_w < 0 || pad_h >= kh || pad_w >= kw)
    return arg_error("max_pool2d_i8");
  // every window must touch the input, otherwise the int32 result (INT32_MIN) has no int8 form
  if ((oh - 1) * stride_h - pad_h >= h || (ow - 1) * stride_w - pad_w >= w) return arg_error("max_pool2d_i8 window");
  if (((uintptr_t)xp | (uintptr_t)yp) & 3) return arg_error("max_pool2d_i8 alignment");
  const int cp = pad_channels(c);
  const int64_t npix = (int64_t)n * oh * ow;
  const int64_t total = act_bytes(npix, cp) / 4;
  hipStream_t s = as_stream(stream);
  KernelTimer timer("k_max_pool_i8", (double)n * c * ((double)h * w + (double)oh * ow), s);
  if (cp >= 16) {
    if (((uintptr_t)xp | (uintptr_t)yp) & 15) return arg_error("max_pool2d_i8 alignment");
    const int8_t* x8 = reinterpret_cast<const int8_t*>(xp);
    int8_t* y8 = reinterpret_cast<int8_t*>(yp);
    if ((int64_t)n * h * w >= 0x7fffffff || npix >= 0x7fffffff) return arg_error("max_pool2d_i8 size");
    const FastDiv dow = make_fastdiv((uint32_t)ow), doh = make_fastdiv((uint32_t)oh);
    if ((kh == 3 && kw == 3) || (kh == 2 && kw == 2)) {
      const unsigned grid = grid_for((total / 4 + 1) / 2, 256, 1 << 16);   // two granules per thread
      if (kh == 3)
        k_max_pool_i8x16<3, 3><<<grid, 256, 0, s>>>(x8, y8, total / 4, npix, cp, h, w, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w, dow, doh);
      else
        k_max_pool_i8x16<2, 2><<<grid, 256, 0, s>>>(x8, y8, total / 4, npix, cp, h, w, oh, ow, kh, kw, stride_h, stride_w, pad_h, pad_w, dow, doh);
    } else {
      k_max_pool_i8x16<0, 0><<<grid_for(total / 4, 256, 1 << 16), 256, 0, s>>>(x8, y8, total / 4, npix, cp, h, w, oh, ow, kh, kw,
                                                                                stride_h, stride_w, pad_h, pad_w, dow, doh);
    }
  } else {
    k_max_pool_i8<<<grid_for(total, 256, 1 << 16), 256, 0, s>>>(reinterpret_cast<const uint32_t*>(xp),
                                                              reinterpret_cast<uint32_t*>(yp), total, npix, cp, h, w, oh, ow,
                                                              kh, kw, stride_h, stride_w, pad_h, pad_w);
  }
  return check_launch("max_pool2d_i8");
}

int cvmhip_sum_hw_i8(const void* xp, const cvmhip_chain* chain, void* out, int out_is_i8,
                     int n, int c, int hw, void* stream) {
  if (!xp || !out || n < 1 || c < 1 || hw < 1) return arg_error("sum_hw_i8");
  if (((uintptr_t)xp | (uintptr_t)out) & 3) return arg_error("sum_hw_i8 alignment");
  DevChain ch;
  if (!make_chain(chain, &ch)) return arg_error("sum_hw_i8 chain");
  const int cp = pad_channels(c);
  const int64_t total = act_bytes(n, cp) / 4;
  hipStream_t s = as_stream(stream);
  KernelTimer timer("k_sum_hw_i8", (double)n * c * hw + (double)n * c, s);  // bytes in + out
  k_sum_hw_i8<<<grid_for(total * SUM_LANES, 256), 256, 0, s>>>(reinterpret_cast<const uint32_t*>(xp), out, out_is_i8, total, n, c, cp,
                                                   hw, ch);
  return check_launch("sum_hw_i8");
}

}  // extern "C"
