// Internal interface of the int8 implicit-GEMM convolution (conv_mfma.hip),
// shared by the operator-level C ABI and the fused graph executor.
#ifndef CVM_CONV_MFMA_H_
#define CVM_CONV_MFMA_H_

#include "hip_common.h"

namespace cvmhip {

enum { OUT_I32_NCHW = 0, OUT_I8_ACT = 1 };

// Division of n < 2^31 by a fixed divisor in three instructions (multiply-high,
// add, shift): q = (mulhi(n, m) + n) >> l with l = ceil(log2 d),
// m = floor(2^32 * (2^l - d) / d) + 1.  The kernels decode pixel indices with it;
// a wavefront that runs alone on its SIMD pays full latency for every
// instruction, so the ~40-instruction generic division matters.
struct FastDiv {
  uint32_t m;
  int32_t l;
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.l = 0;
  while ((1u << f.l) < d) ++f.l;
  f.m = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << f.l) - d)) / d + 1);
  return f;
}
__host__ __device__ inline uint32_t fastdiv(uint32_t n, FastDiv f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (__umulhi(n, f.m) + n) >> f.l;
#else
  return (uint32_t)((((uint64_t)n * f.m) >> 32) + n) >> f.l;
#endif
}

struct ConvGeom {
  int N, H, W, Cp;         // input: int8 activations in the layout above, channels padded to Cp
  int C;                   // true channel count (0 = unknown, only used to count algorithmic work)
  int OC, OH, OW;          // output extent
  int KH, KW, SH, SW, PH, PW, DH, DW;
  int taps, K, Kp;         // filled by conv_igemm: KH*KW, taps*Cp, K rounded up to 64
  int64_t P;               // filled by conv_igemm: N*OH*OW
  union {   // the two kernels need different extras; sharing the space keeps the kernel argument block at its size
    struct { int adv_c, adv_tap, adv_r, adv_s; };   // tiled kernel: cursor advance of one K step (channel, tap, filter row/column)
    struct {                                         // wavefront kernel, filled by conv_igemm_ws: K cut into kslices ranges over
      int kslices, slice_shift, slice_stride, slice_chunks;   // the grid (0 or 1 = no; else 2 or 4 = 1 << slice_shift, the slice is
    };                                               // the low bits of the block index), int32 elements from one slice's plane of
                                                     // partial sums to the next, 32-byte chunks of K per slice
  };
  FastDiv div_ohw, div_ow, div_ct, div_kw;  // filled by conv_igemm: division by OH*OW, OW, Cp/32 and KW
  int row_bytes;           // > 0: row-window input (see stem_* below): bytes of K per filter row, 16 or 32
  int dw;                  // 1: depthwise convolution through MFMA -- output channel tile t reads input channels 32t .. 32t+31 only,
                           //    filter packed by pack_depthwise_diag (OC == C, Cp % 32 == 0)
  int octiles;             // filled by conv_igemm for the wavefront kernel: channel tiles of the grid, and division by it
  FastDiv div_octiles;
};

// What happens to an accumulator before it is stored:
//   v = chain(acc + bias[oc]);  if (residual) v = chain2(v + residual[p][oc]);
struct Epilogue {
  const int32_t* bias;     // device pointer or nullptr
  int bias_vec;            // set by conv_igemm: bias is 16-byte aligned
  DevChain chain;
  const int8_t* residual;  // int8 activations with out_cp channels, or nullptr
  DevChain chain2;
  int out_mode;            // OUT_I32_NCHW or OUT_I8_ACT
  int out_cp;              // padded channel count of the int8 output / residual (>= OC)
  // int32 output: element (n, oc, pixel) goes to out[n*o32_img + oc*o32_ch + pixel*o32_px].  All zero
  // (the default) means NCHW, filled in by conv_igemm; {stride, 1, OC} writes NHWC rows of image n at
  // out + n*stride, e.g. straight into its slice of a concatenated tensor.
  int64_t o32_img;
  int o32_ch, o32_px;
  // 1: max_pool2d with a 2x2 window, stride 2 and no padding follows the chain (ops.cc:466-523 for such a window: the
  // maximum of four values that all exist) and is taken before the store: the output tensor is (N, OC, OH/2, OW/2),
  // int8, OH and OW even.  The wavefront and large-tile kernels then enumerate the convolution's pixels window by
  // window (pixel index = 4 * window + 2 * (oh % 2) + ow % 2), so the four values of a window sit in four
  // neighbouring lanes.  Set through conv_igemm_ws only where conv_pool_eligible says so.
  int pool;
  // int32 output over two destinations: two convolutions over the same input with the same geometry and chain (the
  // class and box heads of a detector's feature map) computed as one, the second one's filter rows behind the
  // first one's, which are padded to a multiple of 32.  Output channels [0, split) go to `out` as described above
  // (oc_a of them exist), channels split .. split + oc_b - 1 to out_b with strides of their own.  split == 0: one destination.
  int split, oc_a, oc_b;
  int o32_ch_b, o32_px_b;
  int64_t o32_img_b;
  int32_t* out_b;
  // which parts of which stages of chain / chain2 do anything (chain_flags_of), filled by conv_igemm: one scalar word a
  // kernel branches on instead of comparing the stage parameters themselves (0: not filled, the kernel works them out)
  unsigned chain_flags, chain2_flags;
};
// bit 31: valid; stage t (bits 5t .. 5t+4): exists, multiplies, shifts before the add, adds, shifts after it
__host__ __device__ inline unsigned chain_flags_of(const DevChain& c) {
  unsigned f = 0x80000000u;
  for (int t = 0; t < 4; ++t) {
    if (t >= c.count) break;
    const DevStage& q = c.st[t];
    f |= (1u | (q.mul != 1 ? 2u : 0u) | (q.s1 != 0 ? 4u : 0u) | (q.add != 0 ? 8u : 0u) | (q.s2 != 0 ? 16u : 0u)) << (5 * t);
  }
  return f;
}

// ---- int8 activation layout.  Channels are padded to Cp = 4, 8, 16 or a
// multiple of 32.  Cp <= 16: plain NHWC.  Cp % 32 == 0: "pixel-blocked" -- the
// tensor is cut into blocks of 32 consecutive pixels (linear index over n, h, w)
// x 32 channels, and a block is stored as the 1 KiB a wavefront feeds to
// v_mfma_i32_32x32x32_i8: lane l holds pixel (l & 31), channels (l >> 5)*16 .. +15.
//   offset(p, c) = ((p/32)*(Cp/32) + c/32)*1024 + ((c/16)%2)*512 + (p%32)*16 + c%16
// Any 16 channel-aligned bytes of one pixel are contiguous in both forms, and a
// 1x1 convolution reads its operand as whole contiguous blocks.
__host__ __device__ inline bool act_blocked(int cp) { return (cp & 31) == 0; }
__host__ __device__ inline int64_t act_offset(int64_t p, int c, int cp) {
  if (!act_blocked(cp)) return p * cp + c;
  return ((p >> 5) * (cp >> 5) + (c >> 5)) * 1024 + ((c >> 4) & 1) * 512 + (p & 31) * 16 + (c & 15);
}
__host__ __device__ inline int64_t act_bytes(int64_t npix, int cp) {
  return act_blocked(cp) ? ((npix + 31) & ~(int64_t)31) * cp : npix * cp;
}
// dword i of the buffer -> pixel and first of its 4 channels
__host__ __device__ inline void act_decode(int64_t i, int cp, int64_t* p, int* c) {
  if (!act_blocked(cp)) {
    const int c4n = cp >> 2;
    *p = i / c4n;
    *c = (int)(i - *p * c4n) * 4;
  } else {
    const int ctiles = cp >> 5;
    const int64_t blk = i >> 8;
    const int w = (int)(i & 255);
    // one division per element of a bandwidth kernel: a shift when the channel tile count is a power of two (the usual
    // case), a 32-bit division when the block index fits, the 64-bit one (some sixty instructions) only otherwise
    const unsigned ct = (unsigned)ctiles;
    int64_t ptile;
    if ((ct & (ct - 1)) == 0) ptile = blk >> (31 - __builtin_clz(ct));
    else if (blk <= 0xffffffffll) ptile = (int64_t)((uint32_t)blk / ct);
    else ptile = blk / ctiles;
    *p = ptile * 32 + ((w >> 2) & 31);
    *c = (int)(blk - ptile * ctiles) * 32 + (w >> 7) * 16 + (w & 3) * 4;
  }
}

// ---- max_pool2d on int8 activations: one 16-byte granule (16 channels of one output pixel).  The window's taps are
// all requested before the first one is used (KH, KW are compile-time: with a loop over a run-time window every
// tap waits for its own trip to memory, nine in a row for a 3x3 window).  A tap outside the image reads the nearest
// pixel inside it instead, which belongs to the same window because every window touches the image (checked by the
// host), so it changes no maximum and the loads need no predicate.  Bytes are compared two at a time as 16-bit
// lanes (even bytes shifted up, odd bytes in place, low halves zero: the order of the signed bytes is kept).
#if defined(__HIPCC__)
typedef short pool_v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pool_max16(uint32_t a, uint32_t b) {
  const pool_v2s r = __builtin_elementwise_max(__builtin_bit_cast(pool_v2s, a), __builtin_bit_cast(pool_v2s, b));
  return __builtin_bit_cast(uint32_t, r);
}
template <int KH, int KW, typename Load>
__device__ __forceinline__ void max_pool_request(int4 (&v)[KH * KW], Load load, int n, int p, int q, int c0, int cp, int h, int w, int sh,
                                                 int sw, int ph, int pw) {
#pragma unroll
  for (int r = 0; r < KH; ++r) {
    int ih = p * sh + r - ph;
    ih = ih < 0 ? 0 : (ih > h - 1 ? h - 1 : ih);
#pragma unroll
    for (int c = 0; c < KW; ++c) {
      int iw = q * sw + c - pw;
      iw = iw < 0 ? 0 : (iw > w - 1 ? w - 1 : iw);
      v[r * KW + c] = load(act_offset((int64_t)(n * h + ih) * w + iw, c0, cp));
    }
  }
}
template <int NT>
__device__ __forceinline__ int4 max_pool_reduce(const int4 (&v)[NT]) {
  uint32_t ev[4], od[4];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const uint32_t d[4] = {(uint32_t)v[t].x, (uint32_t)v[t].y, (uint32_t)v[t].z, (uint32_t)v[t].w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t e = (d[k] << 8) & 0xff00ff00u, o = d[k] & 0xff00ff00u;
      ev[k] = t == 0 ? e : pool_max16(ev[k], e);
      od[k] = t == 0 ? o : pool_max16(od[k], o);
    }
  }
  return make_int4((int)(od[0] | (ev[0] >> 8)), (int)(od[1] | (ev[1] >> 8)), (int)(od[2] | (ev[2] >> 8)), (int)(od[3] | (ev[3] >> 8)));
}
#endif

// Forced kernel choice of the calling thread (thread-local; automatic by default): which implicit-GEMM kernel,
// which configuration of the wavefront kernel (-1 = automatic), which tile of the tiled kernel (0 = automatic).
enum { CONV_KERNEL_AUTO = 0, CONV_KERNEL_LDS = 1, CONV_KERNEL_WAVE = 2, CONV_KERNEL_BIG = 3 };
struct ConvTuning {
  int kernel, wave_cfg, tile_wm, tile_wn;
  // layer-sequence launches: polls after which a wait at a layer boundary gives up
  int seq_spin_limit;
  unsigned long long* seq_stamps;   // device memory for time stamps inside sequence launches (nullptr: none), see CVM_SEQ_STAMP
  int seq_stamp_layers;             // layers it has room for: 256 workgroups x layers x 8 words
  signed char seq_layer_cfg[64];    // configuration forced for entry i of the next sequence tables (-1: automatic)
  int seq_chains;                   // 1: conv_seq_link may chain 1x1 layers behind the layer that feeds them
};
void set_conv_tuning(const ConvTuning& t);

int pad_channels(int c);
size_t packed_act_bytes(int64_t npix, int c);

// ---- row-window form of a convolution over a few input channels (the RGB stem).
// The input is stored as int8 [N][Hp][Wp][4], already padded with zeros, so the
// KW taps x 4 channel bytes of one filter row are contiguous in memory; they are
// read as one window of row_bytes = 16 or 32 bytes and K is ordered
// k = kh*row_bytes + kw*4 + c.  No tap is ever outside the stored tensor, so the
// kernel needs neither masks nor per-tap address arithmetic.
struct StemGeom {
  int hp, wp;        // stored (padded) height and width
  int row_bytes;     // 16 or 32
  int k, kp;         // KH*row_bytes, rounded up to 64
  size_t bytes;      // size of the stored input
};
bool stem_eligible(int c, int kh, int kw, int dil_h, int dil_w);
StemGeom stem_geom(int n, int h, int w, int kh, int kw, int sh, int sw, int ph, int pw);
size_t packed_stem_weight_bytes(int oc, int kp);
int pack_stem_input(const int32_t* x, int8_t* xs, int n, int c, int h, int w, int kh, int kw, int sh, int sw, int ph,
                    int pw, hipStream_t s);
int pack_stem_weights(const int32_t* w, int8_t* wp, int oc, int c, int kh, int kw, hipStream_t s);
// Row-window convolution + chain + max_pool2d(3x3, stride 2, padding 1) in one launch (k_stem_pool): xs from
// pack_stem_input, wp from pack_stem_weights, out the pooled int8 tensor (n, oc, qh, qw); oc 32 or 64.
bool stem_pool_eligible(int c, int oc, int kh, int kw, int oh, int ow, int qh, int qw);
int stem_pool(const int8_t* xs, const int8_t* wp, const int32_t* bias, const DevChain& chain, int8_t* out, int n, int c, int h,
              int w, int oc, int kh, int kw, int sh, int sw, int ph, int pw, int qh, int qw, hipStream_t s);
void weight_dims(int oc, int ic, int kh, int kw, int* ocp, int* kp);
size_t packed_weight_bytes(int oc, int ic, int kh, int kw);
// Two filters over the same input packed as one: the first one's 32-row tiles, then the second one's.
size_t packed_weight_pair_bytes(int oc_a, int oc_b, int ic, int kh, int kw);
int pack_weights_pair(const int32_t* w_a, int oc_a, const int32_t* w_b, int oc_b, int8_t* wp, int ic, int kh, int kw, hipStream_t s);

size_t packed_depthwise_diag_bytes(int c, int kh, int kw);
int pack_depthwise_diag(const int32_t* w, int8_t* wp, int c, int kh, int kw, hipStream_t s);
int pack_activations(const int32_t* x, int8_t* xp, int n, int c, int hw, hipStream_t s);
int unpack_activations(const int8_t* xp, int32_t* x, int n, int c, int hw, hipStream_t s);
int pack_weights(const int32_t* w, int8_t* wp, int oc, int ic, int kh, int kw, hipStream_t s);
int conv_igemm(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep, hipStream_t s);
// The same with a workspace: a layer with at most 64 output pixels and K >= 8192 is then computed in K slices by
// several workgroups per tile (partial sums in the workspace, a second kernel finishes).  Without a workspace, or for
// any other layer, identical to conv_igemm.  conv_slices_workspace_bytes() gives the size (0 = not applicable).
size_t conv_slices_workspace_bytes(const ConvGeom& g, const Epilogue& ep);
// Whether a convolution with this geometry (N, H, W, Cp, OC, OH, OW, filter, strides, padding, dilation set) can take
// Epilogue::pool: int8 pixel-blocked input and output (channels padded to 32 on both sides), an even output extent,
// a filter side of at most 32.
bool conv_pool_eligible(const ConvGeom& g);
// Independent convolutions in one launch (k_conv_group / k_conv_group8): table entries of conv_seq_layer_bytes() bytes; the
// entries of one table all have int32 output or all int8 output.
int conv_group_layer(void* table, int index, int first_block, const int8_t* xp, const int8_t* wp, void* out, ConvGeom g,
                     const Epilogue& ep, int* blocks);
int conv_group_launch(const void* dev_table, int nlayers, int total_blocks, int out_is_i8, double ops, double bytes, hipStream_t s);
int conv_igemm_ws(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep, void* ws, size_t ws_bytes,
                  hipStream_t s);

// ---- a run of convolutions in one launch (k_conv_seq): every XCD (of the 8, 4, 2 or 1 that divide the batch) computes all
// layers for its share of the images and layer boundaries are counters in that XCD's L2.  The caller builds a host
// table with conv_seq_layer (one entry per convolution, in order; each must only read tensors that earlier entries
// or earlier launches wrote), copies it to the device and launches it; `sync` is conv_seq_sync_bytes() of zeroed
// device memory, 256-byte aligned, whose last block holds an error flag (non-zero: a wait ran out, results invalid).
// Two sequence launches must never be in flight at once on one device (each needs every compute unit).
size_t conv_seq_layer_bytes();
size_t conv_seq_sync_bytes();
int conv_seq_shares();
int conv_seq_layer(void* table, int index, const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep);
int conv_seq_layer_config(const void* table, int index);   // configuration of the tile kernel chosen for an entry
int conv_seq_layer_chain(const void* table, int index);    // entries chained behind this one (0, 1 or 2), + 16: no boundary behind it
int conv_seq_link(void* table, int count);                 // chains 1x1 layers behind the layer that feeds them; returns the chains found
int conv_seq_launch(const void* dev_table, int nlayers, void* sync, double ops, double bytes, hipStream_t s);

}  // namespace cvmhip
#endif
