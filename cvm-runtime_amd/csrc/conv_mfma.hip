// conv2d / dense on gfx950 as an exact int8 x int8 -> int32 implicit GEMM.
//
//   D[oc][px] = sum_k W[oc][k] * Xcol[px][k],   k = (kh, kw, c),  px = (n, oh, ow)
//
// Data layout: everything that feeds v_mfma_i32_32x32x32_i8 lives in memory in
// the order the instruction wants it ("fragment order": a block of 32 rows x 32
// bytes of K is the 1 KiB where lane l holds row l & 31, bytes (l >> 5)*16..+15).
//   X : int8 activations, pixel-blocked when Cp % 32 == 0, NHWC for Cp = 4, 8, 16
//       (conv_mfma.h: act_offset)
//   W : int8 filter in fragment order, k ordered (kh, kw, c) with c padded to Cp,
//       K padded to 64, OC to 128 (k_pack_weights)
//   D : int32 NCHW (the operator contract) or int8 activations in the layout above
//       (fused requantised output)
//
// Two kernels, same arithmetic (integer sums commute, so they agree bit for bit):
//   k_conv_igemm  workgroup tile (64*WM) x (64*WN), operands staged in LDS in
//                 fragment order (global -> LDS -> MFMA registers are straight
//                 1 KiB block copies for the filter and, for 1x1 convolutions, the
//                 activations), registers prefetch two K steps ahead, one barrier
//                 per step.  Serves every layout and the large layers.
//   k_conv_wave   no LDS and no barrier in the K loop: each wavefront streams its
//                 own fragments from memory, the wavefronts of a workgroup split
//                 K and meet in LDS once.  Serves layers whose grid is too small
//                 to hide the per-step latency of the tiled kernel.
#include <stdlib.h>
#include <string.h>

#include <type_traits>

#include "conv_mfma.h"

namespace cvmhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ int4 zero4() { return make_int4(0, 0, 0, 0); }

// Source of every out-of-image (padding) granule: loads stay unconditional and
// the data needs no fix-up afterwards.
__device__ __attribute__((aligned(16))) int g_zero_granule[4] = {0, 0, 0, 0};  // never written

// clamp(v, lo, hi) for lo <= hi in one instruction
__device__ __forceinline__ int32_t clamp3(int32_t v, int32_t lo, int32_t hi) {
  int32_t r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
  return r;
}

// A requantisation chain over N values held in registers.  The stage parameters are wave-uniform
// (scalar registers), so a stage costs one instruction per value for the clamp and two for the
// rounding shift.  Straight-line code over the (at most four) stages, each part of a stage an update
// in place under a wave-uniform condition: a loop over the stages, or alternative forms of a stage
// that meet at a join, make the compiler copy all N registers from one set to another at every edge
// (measured: 40 % of the vector instructions of an epilogue were such copies).
constexpr int SEQ_MAX_STAGES = 2;   // stages per chain of a layer inside a layer-sequence launch
// `flags` (chain_flags_of, or 0: worked out here) says which parts exist, in one word that is made a scalar: the
// conditions are then scalar bit tests whatever registers the stage parameters themselves arrive in (read from a table
// in LDS they are vector registers, and a comparison of those is a vector compare, a wait for its result and a
// branch -- twenty of them per chain).
// MAXST, MUL: the caller knows that the chain has at most MAXST stages and (MUL false) none that multiplies -- the
// layer-sequence kernel, whose host side admits no other layers: every layer of a sequence executes its epilogue code
// once or twice, straight from memory, and code for stages that never occur is fetched like any other.
template <int N, int MAXST = 4, bool MUL = true>
__device__ __forceinline__ void run_chain(const DevChain& c, int32_t (&v)[N], const unsigned flags = 0u) {
  unsigned f = flags;
  if (!(__builtin_amdgcn_readfirstlane((int)flags) & 0x80000000u)) f = chain_flags_of(c);   // (a branch: the forty instructions are skipped)
  f = (unsigned)__builtin_amdgcn_readfirstlane((int)f);
#pragma unroll
  for (int t = 0; t < MAXST; ++t) {
    if (f & (1u << (5 * t))) {
      const DevStage q = c.st[t];
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = clamp3(v[e], q.lo, q.hi);
      if (MUL && (f & (2u << (5 * t)))) {   // a multiplication stage (rare)
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = wmul(v[e], q.mul);
      }
      if (f & (4u << (5 * t))) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = v[e] >> q.s1;
      }
      if (f & (8u << (5 * t))) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = wadd(v[e], q.add);
      }
      if (f & (16u << (5 * t))) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = v[e] >> q.s2;
      }
    }
  }
}

// The same chain read from the structure itself, for kernels that receive it as a kernel argument (one launch per
// layer): every field is then a scalar already and the tests below are scalar branches as they stand, while the flag
// word, its readfirstlane and its bit tests only add to such a kernel (ResNet-50 batch 1 0.2607 -> 0.2562 ms, batch
// 16 with one launch per layer 0.421 -> 0.412 ms; with the bias added in the epilogue as well, 0.2485 and 0.393 ms).
template <int N>
__device__ __forceinline__ void run_chain_plain(const DevChain& c, int32_t (&v)[N]) {
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if (t < c.count) {
      const DevStage q = c.st[t];
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = clamp3(v[e], q.lo, q.hi);
      if (q.mul != 1) {   // a multiplication stage (rare)
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = wmul(v[e], q.mul);
      }
      if (q.s1 != 0) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = v[e] >> q.s1;
      }
      if (q.add != 0) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = wadd(v[e], q.add);
      }
      if (q.s2 != 0) {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = v[e] >> q.s2;
      }
    }
  }
}

// low bytes of four values -> one dword
__device__ __forceinline__ uint32_t pack_bytes(int32_t a, int32_t b, int32_t c, int32_t d) {
  const uint32_t lo2 = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t hi2 = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
  return __builtin_amdgcn_perm(hi2, lo2, 0x05040100u);
}

// a's lanes 32..63 <-> b's lanes 0..31
typedef unsigned v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void half_swap(uint32_t& a, uint32_t& b) {
  const v2u r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r.x;
  b = r.y;
}

// the bias of the workgroup's BM output channels, staged in LDS by the first BM threads
template <int BM>
__device__ __forceinline__ void stage_bias(int* sBias, const Epilogue& ep, int OC, int oc0, int tid) {
  if (tid < BM) sBias[tid] = (ep.bias && oc0 + tid < OC) ? ep.bias[oc0 + tid] : 0;
}

// keeps only the bytes of d[0..N-1] whose channel (first + 4k + byte) is below OC:
// padding channels of the output tensor stay zero whatever the chain maps 0 to
template <int N>
__device__ __forceinline__ void mask_channels(uint32_t (&d)[N], int first, int OC) {
  if (first + 4 * N > OC) {
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const int keep = OC - (first + 4 * k);
      d[k] = keep >= 4 ? d[k] : (keep <= 0 ? 0u : d[k] & ((1u << (8 * keep)) - 1u));
    }
  }
}

// 16 bytes per lane from a tensor that another workgroup of this kernel may have written (COH): the request
// carries device scope, so it is answered by the L2 (the point where the compute units of one XCD meet)
// and never by a line the CU's own L1 kept from an earlier layer.  An offset with its top bit set lies
// outside every buffer (sizes stay below 2^31) and reads as zeros.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
constexpr unsigned kOutsideBuffer = 0x80000000u;
// The base address is the same in every lane and is put into scalar registers explicitly: read from a table in LDS it
// arrives in vector registers, and a memory instruction whose descriptor is not known to be uniform is wrapped into a
// loop over the distinct descriptor values of the lanes (a dozen instructions around every load and store).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t act_rsrc(const void* base) {
  const uintptr_t b = (uintptr_t)base;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(((uintptr_t)hi << 32) | lo), 0, 0x7fffffff, 0x00020000);
}
// `off` is the lane's own offset (the one the descriptor's range check sees), `uni` a wave-uniform one that the
// instruction adds from a scalar register: it costs no vector instruction
template <bool COH>
__device__ __forceinline__ int4 ld16_buf(__amdgpu_buffer_rsrc_t rs, unsigned off, unsigned uni = 0) {
  // (said to be uniform explicitly, for the same reason as the descriptor's base address: computed from a table in LDS)
  const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, __builtin_amdgcn_readfirstlane((int)uni), COH ? 16 : 0);
  return make_int4((int)v[0], (int)v[1], (int)v[2], (int)v[3]);
}
// Stores through a buffer descriptor: a 32-bit offset per lane instead of a 64-bit address, and the instruction is a
// plain vector-memory store whatever the compiler knows about the pointer (a pointer read from a table in LDS is
// "generic" to it and would be stored through with flat instructions, which also count as LDS traffic).
__device__ __forceinline__ void st16_buf(__amdgpu_buffer_rsrc_t rs, unsigned off, const v4i v) {
  __builtin_amdgcn_raw_buffer_store_b128(v4u{(unsigned)v[0], (unsigned)v[1], (unsigned)v[2], (unsigned)v[3]}, rs, (int)off, 0, 0);
}
__device__ __forceinline__ void st8_buf(__amdgpu_buffer_rsrc_t rs, unsigned off, uint32_t a, uint32_t b) {
  typedef unsigned v2u_ __attribute__((ext_vector_type(2)));
  __builtin_amdgcn_raw_buffer_store_b64(v2u_{a, b}, rs, (int)off, 0, 0);
}
__device__ __forceinline__ void st4_buf(__amdgpu_buffer_rsrc_t rs, unsigned off, uint32_t a) {
  __builtin_amdgcn_raw_buffer_store_b32(a, rs, (int)off, 0, 0);
}
__device__ __forceinline__ int4 ld16_l2(__amdgpu_buffer_rsrc_t rs, unsigned off) {
  const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, 16 /* sc1: device scope */);
  return make_int4((int)v[0], (int)v[1], (int)v[2], (int)v[3]);
}

// Epilogue shared by both kernels.  A wavefront holds NG groups of 4 values; group
// u (counted from u0, which is a multiple of NG) belongs to the 32x32 MFMA tile
// t = u / 4 of the wavefront's TM x TN tiles (t = i * TN + j) and is the 4
// consecutive channels q*8 + (lane/32)*4 .. +3, q = u % 4, of pixel lane % 32.
//   v = chain(acc + bias);  if (residual) v = chain2(v + residual);  store
// For a pixel-blocked int8 tensor two half-wave swaps turn the 4 packed dwords of a
// tile into 16 consecutive channels per lane, so the wavefront reads the
// residual and writes the result as one contiguous KiB per tile.
// Residual values of the groups u0 .. u0+NG-1 of a wavefront (same numbering as finish_groups), as
// they lie in memory: for whole tiles the 16 bytes per lane of each tile's KiB block, otherwise the 4
// bytes of each group.  Separate from finish_groups so that a kernel can issue these loads before its
// K loop and find them in registers when the accumulators are ready.
template <int TN, int NG, bool COH = false>
__device__ __forceinline__ void load_residual(uint32_t (&rp)[NG], int u0, int ch_wave, int oc0, int px_wave, int lane,
                                              const ConvGeom& g, const Epilogue& ep) {
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int P = (int)g.P;
  const int ocp = ep.out_cp;
  const bool whole = act_blocked(ocp) && (NG % 4 == 0);
  if (whole) {
#pragma unroll
    for (int t = 0; t < NG / 4; ++t) {
      const int tt = (u0 >> 2) + t;
      const int gj = tt % TN, chb = ch_wave + (tt / TN) * 32;
      // the block exists (all 32 pixel rows of it are allocated) unless it lies past the tensor
      const bool tile_ok = (px_wave + gj * 32) < P && (oc0 + chb) < ocp;
      const int64_t off = ((int64_t)((px_wave >> 5) + gj) * (ocp >> 5) + ((oc0 + chb) >> 5)) * 1024;
      int4 r4 = zero4();
      if constexpr (COH) {
        r4 = ld16_l2(act_rsrc(ep.residual), tile_ok ? (unsigned)off + (unsigned)lane * 16u : kOutsideBuffer);
      } else if (tile_ok) {
        const v4i t4 = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(ep.residual + off + lane * 16));
        r4 = make_int4(t4[0], t4[1], t4[2], t4[3]);
      }
      rp[t * 4] = r4.x; rp[t * 4 + 1] = r4.y; rp[t * 4 + 2] = r4.z; rp[t * 4 + 3] = r4.w;
    }
  } else {
#pragma unroll
    for (int m = 0; m < NG; ++m) {
      const int u = u0 + m, t = u >> 2;
      const int p = px_wave + (t % TN) * 32 + lrow;
      const int oc = oc0 + ch_wave + (t / TN) * 32 + (u & 3) * 8 + lgrp * 4;
      const int64_t roff = act_offset(p < P ? p : 0, oc < ocp ? oc : 0, ocp);
      if constexpr (COH) rp[m] = __builtin_amdgcn_raw_buffer_load_b32(act_rsrc(ep.residual), (int)roff, 0, 16);
      else rp[m] = *reinterpret_cast<const uint32_t*>(ep.residual + roff);
    }
  }
}

// RANGE: only the pixels [p_begin, p_end) are stored (one share of a layer inside the layer-sequence
// kernel); the stores are then ordinary ones, because the next layer reads the tensor from this L2.
// BIASED: the accumulators already hold the bias (the layer-sequence kernel starts them from it), sBias is not read.
// FLAGS: the chains are decoded from their flag words (run_chain) instead of from their fields (run_chain_plain).
template <int TN, int NG, int OUT, bool RANGE = false, bool POOLR = false, bool BIASED = false, bool FLAGS = true>
__device__ __forceinline__ void finish_groups(int32_t (&val)[NG * 4], int u0, const int* sBias, int ch_wave, int oc0,
                                              int px_wave, int lane, void* out, const ConvGeom& g, const Epilogue& ep,
                                              uint32_t (&rp)[NG], int p_begin = 0, int p_end = 0) {
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int P = RANGE ? p_end : (int)g.P;
  const int Plo = RANGE ? p_begin : 0;
  const int ocp = ep.out_cp;
  const bool blocked = act_blocked(ocp);
  // group m: tile (gi, gj), channel quarter gq; ch = first channel inside the workgroup's BM channels
  int gj[NG], ch[NG];
#pragma unroll
  for (int m = 0; m < NG; ++m) {
    const int u = u0 + m;
    const int t = u >> 2;
    gj[m] = t % TN;
    ch[m] = ch_wave + (t / TN) * 32 + (u & 3) * 8 + lgrp * 4;
    if constexpr (!BIASED) {
      const int4 bv = *reinterpret_cast<const int4*>(sBias + ch[m]);
      val[m * 4] = wadd(val[m * 4], bv.x); val[m * 4 + 1] = wadd(val[m * 4 + 1], bv.y);
      val[m * 4 + 2] = wadd(val[m * 4 + 2], bv.z); val[m * 4 + 3] = wadd(val[m * 4 + 3], bv.w);
    }
  }
  // byte offset of the KiB block (pixel block, 32 channels) that tile of group m belongs to
  auto block_off = [&](int m) {
    const int pblk = (px_wave >> 5) + gj[m];
    const int cblk = (oc0 + (ch[m] - lgrp * 4)) >> 5;
    return ((int64_t)pblk * (ocp >> 5) + cblk) * 1024;
  };
  const bool whole = blocked && (NG % 4 == 0);   // whole tiles: 16 bytes per lane
  const bool halves = blocked && NG == 2;         // half a tile (q pair): 8 bytes per lane

  // Fused 2x2 max-pool between registers (Epilogue::pool == 2; the host sets it only for tiles of four pixel blocks, a
  // pixel-blocked int8 output, no residual and a chain that never decreases when its input grows): the window's
  // four values are the same register of the tile's four blocks, so the maximum costs three quarters of an
  // instruction a value, and chain, packing and store then work on a quarter of the values.  Adding the bias first
  // keeps the reference's wrap-around sum; taking the maximum before a non-decreasing chain changes no result.
  // (POOLR is a template argument: the same code behind a run-time test made the ordinary epilogue of every
  // four-block tile slower -- ResNet-50's input layer went from 10 to 30 us)
  if constexpr (POOLR && !RANGE && OUT == OUT_I8_ACT && TN == 4 && NG % 16 == 0) {
    {
      int8_t* y8p = reinterpret_cast<int8_t*>(out);
#pragma unroll
      for (int i = 0; i < NG / 16; ++i) {
        int32_t red[16];
#pragma unroll
        for (int qe = 0; qe < 16; ++qe) {
          const int32_t a = val[(i * 4 + 0) * 16 + qe], b = val[(i * 4 + 1) * 16 + qe], c = val[(i * 4 + 2) * 16 + qe],
                        d = val[(i * 4 + 3) * 16 + qe];
          const int32_t ab = a > b ? a : b, cd = c > d ? c : d;
          red[qe] = ab > cd ? ab : cd;
        }
        if constexpr (FLAGS) run_chain(ep.chain, red, ep.chain_flags);
        else run_chain_plain(ep.chain, red);
        uint32_t a = pack_bytes(red[0], red[1], red[2], red[3]), b = pack_bytes(red[4], red[5], red[6], red[7]),
                 c = pack_bytes(red[8], red[9], red[10], red[11]), d = pack_bytes(red[12], red[13], red[14], red[15]);
        half_swap(a, c);
        half_swap(b, d);
        uint32_t w[4] = {a, c, b, d};
        const int tile_first = oc0 + ch_wave + ((u0 >> 4) + i) * 32;
        const int first = tile_first + lgrp * 16;
        if (tile_first + 32 > g.OC) mask_channels(w, first, g.OC);
        const int window = (px_wave >> 2) + lrow;   // px_wave is a multiple of 128: 32 windows per wavefront tile
        if (px_wave < P && first < ocp) {
          const v4i pk4 = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
          __builtin_nontemporal_store(pk4, reinterpret_cast<v4i*>(y8p + act_offset(window, first, ocp)));
        }
      }
      return;
    }
  }
  // one copy of each step, the residual part an update in place under a uniform condition (two
  // alternative paths that meet again cost a register-to-register copy of every value)
  constexpr int MAXST = RANGE ? SEQ_MAX_STAGES : 4;   // RANGE: a layer of a sequence (conv_seq_layer admits short chains only)
  if constexpr (FLAGS) run_chain<NG * 4, MAXST, !RANGE>(ep.chain, val, ep.chain_flags);
  else run_chain_plain(ep.chain, val);
  if (ep.residual) {   // rp holds what load_residual fetched
    if (whole) {
#pragma unroll
      for (int t = 0; t < NG / 4; ++t) {
        uint32_t a = rp[t * 4], b = rp[t * 4 + 1], c = rp[t * 4 + 2], d = rp[t * 4 + 3];
        half_swap(a, b);
        half_swap(c, d);
        rp[t * 4] = a; rp[t * 4 + 1] = c; rp[t * 4 + 2] = b; rp[t * 4 + 3] = d;
      }
    }
#pragma unroll
    for (int e = 0; e < NG * 4; ++e) val[e] = wadd(val[e], (int32_t)(int8_t)(rp[e >> 2] >> (8 * (e & 3))));
    if constexpr (FLAGS) run_chain<NG * 4, MAXST, !RANGE>(ep.chain2, val, ep.chain2_flags);
    else run_chain_plain(ep.chain2, val);
  }

  if (OUT == OUT_I32_NCHW) {
    const int OHW = g.OH * g.OW;
#pragma unroll
    for (int m = 0; m < NG; ++m) {
      const int p = px_wave + gj[m] * 32 + lrow;
      if (p >= P || p < Plo) continue;
      const int n = (int)fastdiv((unsigned)p, g.div_ohw);
      const int rem = p - n * OHW;
      int oc = oc0 + ch[m];
      // two destinations (Epilogue::split, a multiple of 32, so the four channels of a group share one)
      const bool second = ep.split > 0 && oc >= ep.split;
      oc = second ? oc - ep.split : oc;
      const int limit = second ? ep.oc_b : (ep.split > 0 ? ep.oc_a : g.OC);
      const int o_ch = second ? ep.o32_ch_b : ep.o32_ch;
      int32_t* y32 = second ? ep.out_b + (int64_t)n * ep.o32_img_b + (int64_t)oc * ep.o32_ch_b + (int64_t)rem * ep.o32_px_b
                            : reinterpret_cast<int32_t*>(out) + (int64_t)n * ep.o32_img + (int64_t)oc * ep.o32_ch + (int64_t)rem * ep.o32_px;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (oc + e < limit) y32[(int64_t)e * o_ch] = val[m * 4 + e];
    }
    return;
  }
  int8_t* y8 = reinterpret_cast<int8_t*>(out);
  // Fused 2x2 max-pool (host: only with a pixel-blocked output): the four pixels of a window are the four lanes of a
  // quad, so two quad permutes leave the window's maximum in each of them; lane 0 of the quad stores it as pixel
  // p / 4 of the pooled tensor.
  bool pool = false;
  if constexpr (!RANGE) pool = blocked && ep.pool != 0;
  const bool store_lane = !pool || (lrow & 3) == 0;
  const int pshift = pool ? 2 : 0;
  if (pool) {
#pragma unroll
    for (int e = 0; e < NG * 4; ++e) {
      int32_t v = val[e];
      const int32_t a = __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
      v = v > a ? v : a;
      const int32_t b = __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);   // quad_perm [2, 3, 0, 1]
      val[e] = v > b ? v : b;
    }
  }
  uint32_t pk[NG];
#pragma unroll
  for (int m = 0; m < NG; ++m) pk[m] = pack_bytes(val[m * 4], val[m * 4 + 1], val[m * 4 + 2], val[m * 4 + 3]);
  if (whole) {
#pragma unroll
    for (int t = 0; t < NG / 4; ++t) {
      uint32_t a = pk[t * 4], b = pk[t * 4 + 1], c = pk[t * 4 + 2], d = pk[t * 4 + 3];
      half_swap(a, c);   // lower half wave: channels 0..15 of the tile, upper: 16..31
      half_swap(b, d);
      uint32_t w[4] = {a, c, b, d};
      const int tile_first = oc0 + ch_wave + ((u0 >> 2) + t) / TN * 32;   // same for every lane
      const int first = tile_first + lgrp * 16;
      if (tile_first + 32 > g.OC) mask_channels(w, first, g.OC);          // only the last tile of a ragged channel count
      const int p = px_wave + gj[t * 4] * 32 + lrow;
      if (p < P && p >= Plo && first < ocp) {
        const v4i pk4 = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        if constexpr (RANGE) {
          st16_buf(act_rsrc(y8), (unsigned)block_off(t * 4) + (unsigned)lane * 16u, pk4);   // the tensor is smaller than 2^31 bytes (host)
        } else if (pool) {   // window p / 4 of the pooled tensor, the 16 channels this lane holds
          if ((lrow & 3) == 0) __builtin_nontemporal_store(pk4, reinterpret_cast<v4i*>(y8 + act_offset(p >> 2, first, ocp)));
        } else {
          __builtin_nontemporal_store(pk4, reinterpret_cast<v4i*>(y8 + block_off(t * 4) + lane * 16));
        }
      }
    }
  } else if (halves) {
    uint32_t a = pk[0], b = pk[1];
    half_swap(a, b);     // lower half wave: channels 0..7 of the 16-channel granule, upper: 8..15
    uint32_t w[2] = {a, b};
    const int first = oc0 + ch[0] - lgrp * 4 + lgrp * 8;
    mask_channels(w, first, g.OC);
    const int p = px_wave + gj[0] * 32 + lrow;
    if (p < P && p >= Plo && first < ocp && store_lane) {
      if constexpr (RANGE) st8_buf(act_rsrc(y8), (unsigned)act_offset(p >> pshift, first, ocp), w[0], w[1]);
      else *reinterpret_cast<uint2*>(y8 + act_offset(p >> pshift, first, ocp)) = make_uint2(w[0], w[1]);
    }
  } else {
#pragma unroll
    for (int m = 0; m < NG; ++m) {
      uint32_t w[1] = {pk[m]};
      const int first = oc0 + ch[m];
      mask_channels(w, first, g.OC);
      const int p = px_wave + gj[m] * 32 + lrow;
      if (p < P && p >= Plo && first < ocp && store_lane) {
        if constexpr (RANGE) st4_buf(act_rsrc(y8), (unsigned)act_offset(p >> pshift, first, ocp), w[0]);
        else *reinterpret_cast<uint32_t*>(y8 + act_offset(p >> pshift, first, ocp)) = w[0];
      }
    }
  }
}

// Fetch the 16 consecutive k-bytes of one im2col row that start at filter tap
// (r, s), channel c0.  G = bytes that are contiguous in memory for one filter
// tap: 16 when Cp % 16 == 0, else Cp itself (4 or 8) and the granule spans 16/G taps.
// img_pix = linear pixel index of the image's first pixel.
template <int G>
__device__ __forceinline__ int4 fetch_act(const int8_t* __restrict__ xp, const ConvGeom& g, bool row_ok, int img_pix,
                                          int ih0, int iw0, int tap, int r, int s, int c0) {
  const int8_t* zero = reinterpret_cast<const int8_t*>(g_zero_granule);
  if (G == 16) {
    const int ih = ih0 + r * g.DH, iw = iw0 + s * g.DW;
    const bool ok = row_ok && tap < g.taps && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
    const int8_t* src = ok ? xp + act_offset(img_pix + ih * g.W + iw, c0, g.Cp) : zero;
    return *reinterpret_cast<const int4*>(src);
  } else {
    int v[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16 / G; ++j) {
      const int t = tap + j;
      const int rr = t / g.KW, ss = t - rr * g.KW;
      const int ih = ih0 + rr * g.DH, iw = iw0 + ss * g.DW;
      const bool ok = row_ok && t < g.taps && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
      const int8_t* src = ok ? xp + (int64_t)(img_pix + ih * g.W + iw) * g.Cp : zero;
      if (G == 4) {
        v[j] = *reinterpret_cast<const int*>(src);
      } else {
        const int2 u = *reinterpret_cast<const int2*>(src);
        v[2 * j] = u.x;
        v[2 * j + 1] = u.y;
      }
    }
    return make_int4(v[0], v[1], v[2], v[3]);
  }
}

// XCD-aware tile order.  Workgroups are dealt round-robin to the 8 XCDs (workgroup w runs on XCD w % 8), and each XCD
// has an L2 of its own, so the tiles are renumbered to give every XCD one contiguous run of them: neighbouring tiles
// (the channel tiles of the same pixels, then the next pixels) share their operands in that XCD's L2.  Any grid size:
// XCD x holds ceil((nb - x) / 8) workgroups, its run starts after those of the XCDs before it.
__device__ __forceinline__ int xcd_tile_order(int pid, int nb) {
  const int x = pid & 7, per = nb >> 3, extra = nb & 7;
  return x * per + (x < extra ? x : extra) + (pid >> 3);
}

template <int WM, int WN, int G, int KS, int OUT>
__global__ void __launch_bounds__(256)
k_conv_igemm(const int8_t* __restrict__ xp, const int8_t* __restrict__ wp, void* __restrict__ out,
             const ConvGeom g, const Epilogue ep) {
  constexpr int BM = 64 * WM;        // output channels per workgroup
  constexpr int BN = 64 * WN;        // output pixels per workgroup
  constexpr int CH32 = KS / 32;      // 32-byte chunks of K per step
  constexpr int NA = BM * KS / 4096; // 16-byte granules per thread and K step, filter
  constexpr int NB = BN * KS / 4096; //   ... activations
  // two buffers of each operand in fragment order: granule index = ((tile32*CH32 + chunk)*64 + lane)
  __shared__ __attribute__((aligned(16))) int8_t smem[2 * (BM + BN) * KS];
  int8_t* sA = smem;
  int8_t* sB = smem + 2 * BM * KS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = lane & 31;
  const int lgrp = lane >> 5;

  const int nb = gridDim.x;
  const int pid = xcd_tile_order(blockIdx.x, nb);
  const int oc_tiles = (g.OC + BM - 1) / BM;
  const int oc0 = (pid % oc_tiles) * BM;
  const int64_t px0 = (int64_t)(pid / oc_tiles) * BN;

  // ---- per-thread fetch assignment.  Granule tid + 256*i of an operand: lane
  // part (tid & 63) = row (tid & 31) and 16-byte half (tid >> 5) & 1; wave + 4*i
  // enumerates (32-row tile, chunk).  The 16-byte K column of a thread is fixed.
  const int chunk = wave % CH32;
  const int kc = chunk * 2 + lgrp;
  const int OHW = g.OH * g.OW;
  bool row_ok[NB];
  int img_pix[NB], ih0[NB], iw0[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int64_t p = px0 + ((wave + 4 * i) / CH32) * 32 + lrow;
    row_ok[i] = p < g.P;
    const int pp = row_ok[i] ? (int)p : 0;
    const int n = (int)fastdiv((unsigned)pp, g.div_ohw);
    const int rem = pp - n * OHW;
    const int oh = (int)fastdiv((unsigned)rem, g.div_ow), ow = rem - oh * g.OW;
    img_pix[i] = n * g.H * g.W;
    ih0[i] = oh * g.SH - g.PH;
    iw0[i] = ow * g.SW - g.PW;
  }
  const int nch1 = g.Kp / 32 + 1;
  int wrow[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) wrow[i] = ((oc0 / 32 + (wave + 4 * i) / CH32) * nch1 + chunk) * 1024 + lane * 16;

  // position of this thread's granule inside the (tap, channel) space
  int tap = (kc * 16) / g.Cp, c0 = kc * 16 - tap * g.Cp;
  int r = tap / g.KW, s = tap - r * g.KW;
  int kbyte = 0;

  // Accumulator element e of lane l in a 32x32 tile is row (e/4)*8 + (l/32)*4 + e%4
  // (output channel), column l%32 (pixel).
  __shared__ __attribute__((aligned(16))) int sBias[BM];
  stage_bias<BM>(sBias, ep, g.OC, oc0, tid);   // visible after the first barrier of the K loop
  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // One K step of operands held in registers as a single SSA vector value
  // (granules 0..NA-1 filter, NA..NA+NB-1 activations); two of them are in flight.
  typedef int regs_t __attribute__((ext_vector_type(4 * (NA + NB))));
  const int nk = g.Kp / KS;

  // loads the next K step and advances the (tap, channel) cursor
  auto fetch = [&]() -> regs_t {
    regs_t R;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int4 v = *reinterpret_cast<const int4*>(wp + wrow[i] + kbyte);
      R[4 * i] = v.x; R[4 * i + 1] = v.y; R[4 * i + 2] = v.z; R[4 * i + 3] = v.w;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int4 v = fetch_act<G>(xp, g, row_ok[i], img_pix[i], ih0[i], iw0[i], tap, r, s, c0);
      R[4 * (NA + i)] = v.x; R[4 * (NA + i) + 1] = v.y; R[4 * (NA + i) + 2] = v.z; R[4 * (NA + i) + 3] = v.w;
    }
    kbyte += CH32 * 1024;
    if (G == 16) {
      // advance the cursor by KS bytes without a loop (lanes sit at different granules)
      c0 += g.adv_c;
      const int carry = c0 >= g.Cp ? 1 : 0;
      c0 -= carry ? g.Cp : 0;
      tap += g.adv_tap + carry;
      s += g.adv_s + carry;
      const int wrap = s >= g.KW ? 1 : 0;
      s -= wrap ? g.KW : 0;
      r += g.adv_r + wrap;
    } else {
      tap += KS / G;
    }
    return R;
  };
  auto stage = [&](const regs_t R, int buf) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
      *reinterpret_cast<int4*>(&sA[buf * BM * KS + (tid + 256 * i) * 16]) =
          make_int4(R[4 * i], R[4 * i + 1], R[4 * i + 2], R[4 * i + 3]);
#pragma unroll
    for (int i = 0; i < NB; ++i)
      *reinterpret_cast<int4*>(&sB[buf * BN * KS + (tid + 256 * i) * 16]) =
          make_int4(R[4 * (NA + i)], R[4 * (NA + i) + 1], R[4 * (NA + i) + 2], R[4 * (NA + i) + 3]);
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < CH32; ++ks) {
      v4i a[WM], b[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[i] = *reinterpret_cast<const v4i*>(&sA[buf * BM * KS + (((wm * WM + i) * CH32 + ks) * 64 + lane) * 16]);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j] = *reinterpret_cast<const v4i*>(&sB[buf * BN * KS + (((wn * WN + j) * CH32 + ks) * 64 + lane) * 16]);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  };

  // K step kt: the register set of that parity receives step kt+2, LDS buffer
  // kt&1 is consumed, the other register set (step kt+1, fetched one step
  // earlier) moves to the other LDS buffer.  Fetches are unconditional -- a step
  // past the end reads valid memory (the filter has slack behind it, taps past
  // the filter read the zero granule) and is never consumed -- because a
  // conditional fetch makes the compiler wait for all outstanding loads at the join.
  regs_t R0 = fetch();
  regs_t R1 = fetch();
  stage(R0, 0);
  __syncthreads();
  for (int kt = 0; kt < nk; kt += 2) {
    R0 = fetch();
    mma(0);
    stage(R1, 1);
    __syncthreads();
    if (kt + 1 >= nk) break;
    R1 = fetch();
    mma(1);
    stage(R0, 0);
    __syncthreads();
  }

  // ---- epilogue
  int32_t val[WM * WN * 16];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) val[(i * WN + j) * 16 + e] = acc[i][j][e];
  uint32_t rp[WM * WN * 4];
  if (ep.residual) load_residual<WN, WM * WN * 4>(rp, 0, wm * WM * 32, oc0, (int)px0 + wn * WN * 32, lane, g, ep);
  finish_groups<WN, WM * WN * 4, OUT>(val, 0, sBias, wm * WM * 32, oc0, (int)px0 + wn * WN * 32, lane, out, g, ep, rp);
}

// Bit t set when filter tap t (of k <= 32) of a receptive field that starts at input coordinate x0
// lies inside [0, extent).  Without dilation the valid taps are the run max(0, -x0) ..
// min(k - 1, extent - 1 - x0), which needs no loop and no branch.
// Image and output coordinates of output pixel index p.  Ordinary order: p = (n * OH + oh) * OW + ow.  With a fused 2x2
// max-pool (Epilogue::pool) the pixels are numbered window by window, p = 4 * window + 2 * (oh % 2) + ow % 2 with
// window = (n * OH/2 + oh/2) * OW/2 + ow/2, and the host has set div_ohw and div_ow to divide by OH*OW/4 and OW/2.
// pool == 2 (wavefront tiles of four pixel blocks, pixel count a multiple of 128): the four pixels of a window lie in
// the four blocks of a wavefront's tile at the same lane, p = 128 * (window / 32) + 32 * sub + window % 32, so the
// maximum is taken between registers.
__device__ __forceinline__ void conv_out_pixel(const ConvGeom& g, const int pool, const unsigned p, int& n, int& oh, int& ow) {
  const int OHW = g.OH * g.OW;
  if (!pool) {
    n = (int)fastdiv(p, g.div_ohw);
    const int rem = (int)p - n * OHW;
    oh = (int)fastdiv((unsigned)rem, g.div_ow);
    ow = rem - oh * g.OW;
  } else {
    const unsigned q = pool == 2 ? ((p >> 7) << 5) | (p & 31u) : p >> 2;
    const unsigned sub = pool == 2 ? (p >> 5) & 3u : p & 3u;
    n = (int)fastdiv(q, g.div_ohw);
    const int rem = (int)q - n * (OHW >> 2);
    const int qh = (int)fastdiv((unsigned)rem, g.div_ow);
    const int qw = rem - qh * (g.OW >> 1);
    oh = 2 * qh + (int)(sub >> 1);
    ow = 2 * qw + (int)(sub & 1u);
  }
}

__device__ __forceinline__ unsigned tap_mask_dense(int x0, int extent, int k) {
  int lo = x0 < 0 ? -x0 : 0;
  int hi = extent - 1 - x0;
  hi = hi < k - 1 ? hi : k - 1;
  const bool any = hi >= lo;
  lo = lo < 31 ? lo : 31;
  hi = hi > 0 ? hi : 0;
  const unsigned m = ((2u << hi) - 1u) & ~((1u << lo) - 1u);
  return any ? m : 0u;
}
__device__ __forceinline__ unsigned tap_mask_dilated(int x0, int extent, int k, int d) {
  unsigned m = 0;
  for (int t = 0; t < k; ++t) m |= ((unsigned)(x0 + t * d) < (unsigned)extent ? 1u : 0u) << t;
  return m;
}

// ---------------------------------------------------------------- wavefront-private kernel
// Layers whose grid is small (few pixels, deep K) are bound by latency, not by
// MFMA rate: with one wavefront per SIMD every instruction pays its full
// pipeline latency and every K step of the tiled kernel pays a global -> LDS ->
// barrier round trip.  This kernel has no LDS and no barrier in its K loop:
// every wavefront streams its own operands straight from memory into MFMA
// registers (filter and pixel-blocked activations are both stored in fragment
// order, so a load is 16 bytes per lane and, for a 1x1 convolution, 1 KiB
// contiguous per wavefront) and keeps two batches of D chunks (32 bytes of K
// each) in flight.  The NW wavefronts of a workgroup split the K range KSPLIT
// ways and the pixel axis NW/KSPLIT ways; partial sums meet in LDS once, after
// the loop.  Requires Cp % 32 == 0 (pixel-blocked input; a chunk never
// straddles two filter taps).
//   MODE WAVE_IDENT  1x1, stride 1, no padding: the operand of output pixel block
//                    t is input block t, addresses are base + chunk * 1 KiB
//        WAVE_NOPAD  no padding: every tap of a valid output pixel is inside the image
//        WAVE_ROWS   row-window input of a few-channel convolution (conv_mfma.h: StemGeom):
//                    a chunk is 32 bytes of one or two filter rows, always inside the stored tensor
//        WAVE_PAD    padding: per-lane row / column validity masks (KH, KW <= 32),
//                    out-of-image granules are read from a zero granule
enum { WAVE_IDENT = 0, WAVE_NOPAD = 1, WAVE_PAD = 2, WAVE_ROWS = 3 };

struct alignas(16) SeqLayer {
  const int8_t* xp;
  const int8_t* wf;
  void* out;
  ConvGeom g;
  Epilogue ep;
  int kernel;          // configuration * 3 + mode (identity, no padding, padding)
  int px_per_share;    // output pixels of one share of the images
  int ptiles;          // pixel tiles that cover a share (its first block may begin before the share)
  int shares;          // XCDs that take part: the largest of 1, 2, 4, 8 that divides the batch; the others leave at once
  int chain;           // 1 or 2: the next one or two entries are 1x1 layers over this layer's output pixels, computed by the
                       // same wavefront from registers (conv_chain_tail); they are then not layers of their own
  int join_next;       // 1: the layer behind this one (and its chain) reads nothing that this one writes and writes nothing
                       // that this one touches: no layer boundary between the two
};
constexpr int SEQ_SHARES = 8, SEQ_WG_PER_SHARE = 32, SEQ_SYNC_WORDS = 64;   // counters of a share: one 256-byte line
enum { SEQ_ARRIVE = 0, SEQ_BAR = 1, SEQ_DONE = 2 };

// One tile set of the wavefront-private kernel: workgroup-level tile `pid` (channel tile fastest) of the
// pixel range [p_begin, p_end) (COH only; otherwise the whole layer), computed by the NW wavefronts whose thread index is `tid`, with
// sPart / sBias their LDS.  k_conv_wave is this function over a grid; the layer-sequence kernel calls it
// from its loop over layers with COH set (operands written earlier in the same launch).
// Layer boundary of the layer-sequence kernel, seen from the layer that follows: its wavefronts compute their
// addresses and request their filter operands first, and only then wait here until every workgroup of the
// XCD has counted itself out of the previous layer -- the filter does not depend on that layer, so its trip
// from memory overlaps the wait.  The wait is bounded; when it runs out, or another one has, the error word is
// set and the wavefront goes on (the results are then void, and every later wait ends after 1024 polls).
struct LayerGate {
  unsigned* counter;   // nullptr: nothing to wait for
  unsigned target;
  unsigned* error;
  int spin_limit;
  unsigned* seen;      // LDS word of the workgroup (or of its half): the highest target its first wavefront has seen reached
};
__device__ __forceinline__ void gate_poll(const LayerGate& gate) {
  if (!gate.counter) return;
  unsigned v = __builtin_amdgcn_readfirstlane(__hip_atomic_load(gate.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  int spins = 0;
  if (v < gate.target && gate.spin_limit <= 0) {   // no patience at all (the host's test of its fall-back): give up at once
    __hip_atomic_store(gate.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
  while (v < gate.target) {
    __builtin_amdgcn_s_sleep(1);
    v = __builtin_amdgcn_readfirstlane(__hip_atomic_load(gate.counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    if ((++spins & 1023) == 0) {
      const unsigned e = __builtin_amdgcn_readfirstlane(__hip_atomic_load(gate.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      if (e != 0 || spins > gate.spin_limit) {
        __hip_atomic_store(gate.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
    }
  }
}
// Only the first wavefront of a workgroup (of each half, when two tiles run side by side) polls the counter in the L2;
// the others watch a word in LDS that it sets when it is through -- also when it gave up, so they never wait for longer
// than it did.  Eight wavefronts of each of the XCD's 32 workgroups polling one address kept that L2 channel busy
// with nothing but polls, in front of the very atomic adds they were waiting for.
__device__ __forceinline__ void gate_wait(const LayerGate& gate, const int wave) {
  if (!gate.counter) return;
  if (wave != 0) {
    while (__builtin_amdgcn_readfirstlane(*reinterpret_cast<volatile unsigned*>(gate.seen)) < gate.target) __builtin_amdgcn_s_sleep(1);
    return;
  }
  gate_poll(gate);
  *reinterpret_cast<volatile unsigned*>(gate.seen) = gate.target;
}

// Optional time stamps of a layer inside a layer-sequence launch (cvmhip_set_seq_stamps): eight 64-bit words per
// workgroup and layer -- 0 tile entered, 1 boundary passed, 2 first operand batch multiplied, 3 K loop done, 4 K-split
// exchange done, 5 epilogue issued, 6 counted out, 7 layer begun -- written by the workgroup's first thread for the
// first tile of the layer.  Only in a build with -DCVM_SEQ_STAMPS (cvm-runtime_amd/build.py: CVM_HIP_DEFINES): even
// behind a null test the stamps cost the kernel a wait for all outstanding loads wherever two paths meet.
#ifdef CVM_SEQ_STAMPS
#define CVM_SEQ_STAMP(i, dep)                                              \
  do {                                                                     \
    if constexpr (COH) {                                                   \
      if (tr) {                                                            \
        asm volatile("" ::"v"(dep));                                       \
        if (tid == 0) tr[i] = __builtin_amdgcn_s_memtime();                \
      }                                                                    \
    }                                                                      \
  } while (0)
#else
#define CVM_SEQ_STAMP(i, dep) do { } while (0)
#endif
// One request: 16 bytes per lane from `gaddr` (any address per lane) to LDS byte lds_base + 16 * lane.  Written as
// assembly on purpose: the compiler then neither counts these requests nor protects LDS reads against them (it would
// wait for every outstanding one before the first ds_read of a step, which undoes the ring); the waits are wait_vm.

typedef int8_t __attribute__((address_space(3))) * lptr_t;
__device__ __forceinline__ void lds_dma16(const void* gaddr, uint32_t lds_base) {
  // (the s_nop is the wait state an instruction that reads M0 needs after a scalar write to it; inside inline assembly
  // nobody inserts it for us)
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gaddr), "s"(lds_base) : "memory");
}

// ---------------------------------------------------------------- 1x1 layers computed from registers
// A 1x1 convolution with stride 1 needs, for a block of 32 pixels, nothing but the same 32 pixels of its input.  When
// a wavefront holds a layer's result for a block of pixels with ALL its channels, the requantised int8 values of a
// 32-channel tile, 16 consecutive channels per lane, are at once the KiB block that is stored and the operand an MFMA
// of the next layer takes for those 32 channels of its K: the next layer can be computed right there, with no trip
// through memory, no other wavefront and no layer boundary.  conv_chain_tail does that for one or two such layers
// behind layer A (whose MT2 accumulator tiles the caller hands over): layer B (any number TB of 32-channel tiles,
// optional residual) one tile at a time -- MT2 MFMAs, requantise, store -- and each finished tile is at once multiplied
// into the MT1 accumulator tiles of layer C (MT1 = 0: no layer C), which are requantised and stored at the end.
// Every result is the one the layers give on their own: the same integer sums, the same chains.
//
// One accumulator tile (32 channels x 32 pixels; element e of a lane: channel (e / 4) * 8 + (lane / 32) * 4 + e % 4 of
// pixel lane % 32) -> v = chain(acc); if (residual) v = chain2(v + residual); int8, 16 consecutive channels per lane.
// `res`: the lane's 16 bytes of the residual tensor's KiB block for the same pixels and channels.
__device__ __forceinline__ v4i requant_tile(const v16i acc, const Epilogue& ep, const int4 res) {
  int32_t val[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) val[e] = acc[e];
  run_chain<16, SEQ_MAX_STAGES, false>(ep.chain, val, ep.chain_flags);
  if (ep.residual) {
    uint32_t a = (uint32_t)res.x, b = (uint32_t)res.y, c = (uint32_t)res.z, d = (uint32_t)res.w;
    half_swap(a, b);
    half_swap(c, d);
    const uint32_t rp[4] = {a, c, b, d};
#pragma unroll
    for (int e = 0; e < 16; ++e) val[e] = wadd(val[e], (int32_t)(int8_t)(rp[e >> 2] >> (8 * (e & 3))));
    run_chain<16, SEQ_MAX_STAGES, false>(ep.chain2, val, ep.chain2_flags);
  }
  uint32_t a = pack_bytes(val[0], val[1], val[2], val[3]), b = pack_bytes(val[4], val[5], val[6], val[7]),
           c = pack_bytes(val[8], val[9], val[10], val[11]), d = pack_bytes(val[12], val[13], val[14], val[15]);
  half_swap(a, c);   // lower half wave: channels 0..15 of the tile, upper: 16..31
  half_swap(b, d);
  return v4i{(int)a, (int)c, (int)b, (int)d};
}
// The filters and biases of a chain's layers are the same for every wavefront, and a wavefront's pixel block uses each of
// their bytes once: fetched per wavefront they were most of its memory traffic (and four 16-byte loads per tile for
// the bias alone).  The workgroup copies them to LDS once per step instead, memory -> LDS without passing registers,
// requested BEFORE the wait at the layer boundary (they do not depend on the previous layer): filter of A at byte 0 of
// the block, B's and C's behind it, as they lie in memory; the biases of B and C in `sBias`.
struct ChainLds {
  const char* w;      // LDS: A's packed filter; B's at w + off_b, C's at w + off_c
  unsigned off_b, off_c;
  const int* bias_b;  // LDS: OC_B words (zeros without a bias), C's OC_C words behind them
  const int* bias_c;
};
__device__ __forceinline__ unsigned filter_bytes(const ConvGeom& g) {
  return (unsigned)(g.OC >> 5) * (unsigned)((g.Kp >> 5) + 1) * 1024u;
}
// all 512 threads; the caller waits (vmcnt(0), barrier) before anyone reads
__device__ __forceinline__ ChainLds chain_stage_operands(const SeqLayer& A, const SeqLayer& B, const SeqLayer* C, int* sPart, int* sBias,
                                                         const int tid) {
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const uint32_t lds_w = (uint32_t)(uintptr_t)(lptr_t)reinterpret_cast<int8_t*>(sPart);
  const uint32_t lds_b = (uint32_t)(uintptr_t)(lptr_t)reinterpret_cast<int8_t*>(sBias);
  const unsigned sz_a = filter_bytes(A.g), sz_b = filter_bytes(B.g), sz_c = C ? filter_bytes(C->g) : 0u;
  auto copy = [&](const int8_t* src_generic, const unsigned bytes, const uint32_t dst) __attribute__((always_inline)) {
    const uintptr_t sb = (uintptr_t)src_generic;
    const int8_t* src = reinterpret_cast<const int8_t*>(((uintptr_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(sb >> 32)) << 32) |
                                                        (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)sb));
    const int blocks = __builtin_amdgcn_readfirstlane((int)((bytes + 1023u) >> 10));
    for (int k = wave; k < blocks; k += 8) {
      if ((unsigned)k * 1024u + (unsigned)lane * 16u < bytes)
        lds_dma16(src + (size_t)k * 1024 + lane * 16, (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + (unsigned)k * 1024u)));
    }
  };
  copy(A.wf, sz_a, lds_w);
  copy(B.wf, sz_b, lds_w + sz_a);
  if (C) copy(C->wf, sz_c, lds_w + sz_a + sz_b);
  const int ocb = B.g.OC, occ = C ? C->g.OC : 0;
  if (B.ep.bias) copy(reinterpret_cast<const int8_t*>(B.ep.bias), (unsigned)ocb * 4u, lds_b);
  else for (int k = tid; k < ocb; k += 512) sBias[k] = 0;
  if (C) {
    if (C->ep.bias) copy(reinterpret_cast<const int8_t*>(C->ep.bias), (unsigned)occ * 4u, lds_b + (unsigned)ocb * 4u);
    else for (int k = tid; k < occ; k += 512) sBias[ocb + k] = 0;
  }
  return ChainLds{reinterpret_cast<const char*>(sPart), sz_a, sz_a + sz_b, sBias, sBias + ocb};
}
// the bias of 32 output channels as an accumulator tile holds them
__device__ __forceinline__ v16i bias_tile(const int* sbias, const int first, const int lgrp) {
  v16i r;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int4 bv = *reinterpret_cast<const int4*>(sbias + first + q * 8 + lgrp * 4);
    r[q * 4] = bv.x; r[q * 4 + 1] = bv.y; r[q * 4 + 2] = bv.z; r[q * 4 + 3] = bv.w;
  }
  return r;
}
// The host has checked (conv_seq_link): A, B and C have whole 32-channel tiles and no padding channels, A has MT2 tiles,
// C has MT1, B reads A's output and C reads B's, pixel for pixel; only B may have a residual; every bias is 16-byte
// aligned; the filters fit the LDS block and the biases sBias; no output overlaps anything another wavefront may still
// read in this layer.
template <int MT2, int MT1>
__device__ __forceinline__ void conv_chain_tail(const v16i (&accA)[MT2][1], const Epilogue& epA, void* outA, const SeqLayer& B,
                                                const SeqLayer* C, const ChainLds& lds, const int px_wave, const int lane,
                                                const int p_begin, const int p_end) {
  if (px_wave >= p_end || px_wave + 32 <= p_begin) return;   // none of this wavefront's pixels belong to the share
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int p = px_wave + lrow;
  const bool mine = p >= p_begin && p < p_end;               // pixels of a neighbouring share are computed and not stored
  const unsigned pblk = (unsigned)px_wave >> 5;
  const unsigned lane16 = (unsigned)lane * 16u;

  v4i b2[MT2];   // A's result: the K chunks of B
  {
    const __amdgpu_buffer_rsrc_t rs = act_rsrc(outA);
#pragma unroll
    for (int i = 0; i < MT2; ++i) {
      b2[i] = requant_tile(accA[i][0], epA, zero4());
      if (mine) st16_buf(rs, (pblk * MT2 + i) * 1024u + lane16, b2[i]);
    }
  }
  const Epilogue& eB = B.ep;
  const int TB = __builtin_amdgcn_readfirstlane(B.g.OC >> 5);
  const unsigned strideB = (unsigned)__builtin_amdgcn_readfirstlane((B.g.Kp >> 5) + 1) * 1024u;   // from one 32-channel tile of the packed filter to the next
  const __amdgpu_buffer_rsrc_t rs_oB = act_rsrc(B.out), rs_res = act_rsrc(eB.residual);
  const bool has_res = eB.residual != nullptr;
  const Epilogue& eC = MT1 > 0 ? C->ep : eB;
  const unsigned strideC = MT1 > 0 ? (unsigned)__builtin_amdgcn_readfirstlane((C->g.Kp >> 5) + 1) * 1024u : 0u;
  const char* wB = lds.w + lds.off_b + lane16;
  const char* wC = lds.w + lds.off_c + lane16;
  constexpr int NC = MT1 > 0 ? MT1 : 1;
  v16i accC[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) accC[i] = bias_tile(lds.bias_c, MT1 > 0 ? i * 32 : 0, lgrp);

  // the one thing tile t of B still needs from memory, requested a tile ahead: its block of the residual
  auto request = [&](const int t) __attribute__((always_inline)) -> int4 {
    return ld16_l2(rs_res, has_res ? (pblk * (unsigned)TB + (unsigned)t) * 1024u + lane16 : kOutsideBuffer);
  };
  auto tile = [&](const int4 res, const int t) __attribute__((always_inline)) {
    v16i a = bias_tile(lds.bias_b, t * 32, lgrp);
#pragma unroll
    for (int c = 0; c < MT2; ++c) {
      const int4 w = *reinterpret_cast<const int4*>(wB + (unsigned)t * strideB + (unsigned)c * 1024u);
      a = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i{w.x, w.y, w.z, w.w}, b2[c], a, 0, 0, 0);
    }
    const v4i b3 = requant_tile(a, eB, res);
    if (mine) st16_buf(rs_oB, (pblk * (unsigned)TB + (unsigned)t) * 1024u + lane16, b3);
    if constexpr (MT1 > 0) {
#pragma unroll
      for (int i = 0; i < MT1; ++i) {
        const int4 w = *reinterpret_cast<const int4*>(wC + (unsigned)i * strideC + (unsigned)t * 1024u);
        accC[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i{w.x, w.y, w.z, w.w}, b3, accC[i], 0, 0, 0);
      }
    }
  };
  // one copy of the tile's code (a second one would double what the instruction cache has to fetch): the block
  // requested ahead changes hands in registers
  int4 r0 = request(0);
  for (int t = 0; t < TB; ++t) {
    const int4 r1 = request(t + 1 < TB ? t + 1 : t);
    tile(r0, t);
    r0 = r1;
  }
  if constexpr (MT1 > 0) {
    const __amdgpu_buffer_rsrc_t rs_oC = act_rsrc(C->out);
#pragma unroll
    for (int i = 0; i < MT1; ++i) {
      const v4i y = requant_tile(accC[i], eC, zero4());
      if (mine) st16_buf(rs_oC, (pblk * MT1 + i) * 1024u + lane16, y);
    }
  }
}

// TAIL >= 0 (layer-sequence kernel, unsplit K, one pixel block per wavefront, all of the layer's channels in the tile): the
// accumulators go to conv_chain_tail<TM, TAIL> with the table entries tailB, tailC instead of the epilogue.
template <int TM, int TN, int KSPLIT, int NW, int D, int OUT, int MODE, bool SLICES, bool COH, bool POOLR = false, int TAIL = -1>
__device__ __forceinline__ void conv_wave_tile(const int8_t* __restrict__ xp, const int8_t* __restrict__ wf, void* __restrict__ out,
                                               const ConvGeom& g, const Epilogue& ep, int pid, const int tid,
                                               int* __restrict__ sPart, int* __restrict__ sBias, const int p_begin = 0,
                                               const int p_end = 0, const LayerGate gate = LayerGate{nullptr, 0, nullptr, 0, nullptr},
                                               unsigned long long* tr = nullptr, const SeqLayer* tailB = nullptr,
                                               const SeqLayer* tailC = nullptr, const ChainLds* chain_lds = nullptr) {
  CVM_SEQ_STAMP(0, tid);
  constexpr int PS = NW / KSPLIT;         // wavefronts side by side along the pixel axis
  constexpr int BM = 32 * TM;             // output channels per workgroup
  constexpr int WPIX = 32 * TN;           // pixels per wavefront
  constexpr int BN = WPIX * PS;           // pixels per workgroup
  constexpr int U = TM * TN * 4;          // groups of 4 accumulator registers (4 consecutive channels) per wavefront
  constexpr int NU = U / KSPLIT;          // groups one wavefront finalises
  static_assert(NW % KSPLIT == 0 && U % KSPLIT == 0, "split must divide the work");
  static_assert(!(COH && (MODE == WAVE_ROWS || SLICES)), "the layer-sequence kernel has no row-window or K-sliced form");

  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kw_ = wave % KSPLIT, pw_ = wave / KSPLIT;
  const int lrow = lane & 31, lgrp = lane >> 5;
  // After a K split a wavefront finalises the groups kw_*NU .. kw_*NU + NU-1 of the workgroup's tile
  // set.  It computes them in its register groups 0 .. NU-1: register group u (tile u / 4, quarter
  // u % 4) holds the workgroup's group u ^ G, G = kw_ * NU.  The own groups then never travel through
  // LDS and every register index is still a constant; the permutation costs nothing, because it only
  // changes addresses: tiles are exchanged by swapping operand pointers (X), quarters of a tile by
  // letting each lane fetch the filter row (lane ^ 8 Q) of its 32-row block.
  const int G = KSPLIT > 1 ? kw_ * NU : 0;
  const int X = G >> 2, Q = G & 3;
  const int Xi = X / TN, Xj = X % TN;

  // K sliced over the grid (g.kslices > 1: a layer with very few tiles and a very long K, whose filter stream
  // needs more workgroups than it has tiles): slice index = low bits of the block index (the slices of a tile then share its activation operand in one L2); a slice writes
  // raw int32 partial sums to its own plane of the workspace and a second kernel adds the planes up.
  // (SLICES: only the instantiation the host launches for such layers carries the code)
  int kslice = 0;
  if (SLICES && g.kslices > 1) {
    kslice = pid & (g.kslices - 1);
    pid >>= g.slice_shift;
  }
  const int ptile = (int)fastdiv((unsigned)pid, g.div_octiles);   // g.octiles = ceil(OC / BM), set by the host for this tile
  const int oc0 = (pid - ptile * g.octiles) * BM;
  const int px0 = (COH ? (p_begin & ~31) : 0) + ptile * BN;   // P < 2^31 is checked on the host
  const int ctiles = g.Cp >> 5;
  const int P = (int)g.P;
  __amdgpu_buffer_rsrc_t rs_x = act_rsrc(xp);   // activations are read through a buffer descriptor: 32-bit offsets, zeros past the end

  // ---- per-lane operand addressing
  unsigned xoff[TN];                       // WAVE_IDENT: byte offset (from xp) of the block's row of this lane
  int rowbase[TN];                         // otherwise: linear index of the first input pixel of the receptive field
  unsigned rowmask[TN], colmask[TN];       // WAVE_PAD: filter rows / columns inside the image
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    if (MODE == WAVE_IDENT) {
      int t = (px0 >> 5) + pw_ * TN + (j ^ Xj);
      const int last = (P - 1) >> 5;
      t = t < last ? t : last;             // blocks past the tensor re-read its last block; their pixels are never stored
      xoff[j] = (unsigned)t * (unsigned)(ctiles * 1024) + (unsigned)lane * 16u;
      rowbase[j] = 0; rowmask[j] = 0; colmask[j] = 0;
    } else {
      const int p = px0 + (pw_ * TN + (j ^ Xj)) * 32 + lrow;
      const bool ok = COH ? (p >= p_begin && p < p_end) : p < P;
      const unsigned pp = ok ? (unsigned)p : 0u;
      int n, oh, ow;
      conv_out_pixel(g, (!COH && MODE != WAVE_ROWS) ? ep.pool : 0, pp, n, oh, ow);
      const int ih0 = oh * g.SH - g.PH, iw0 = ow * g.SW - g.PW;
      rowbase[j] = (n * g.H + ih0) * g.W + iw0;
      if (MODE == WAVE_ROWS) rowbase[j] *= 4;   // byte offset of the window of filter row 0 (g.H, g.W: stored size, no padding left)
      xoff[j] = 0;
      unsigned rm = 0, cm = 0;
      if (MODE == WAVE_PAD) {
        if (g.DH == 1 && g.DW == 1) {
          rm = tap_mask_dense(ih0, g.H, g.KH);
          cm = tap_mask_dense(iw0, g.W, g.KW);
        } else {
          rm = tap_mask_dilated(ih0, g.H, g.KH, g.DH);
          cm = tap_mask_dilated(iw0, g.W, g.KW, g.DW);
        }
        rm = ok ? rm : 0u;
      }
      rowmask[j] = rm;
      colmask[j] = cm;
    }
  }

  // K range of this wavefront, in chunks of 32 bytes; chunks past the true K are never visited
  const int nch = g.Kp >> 5;
  int s_begin = 0, nlive = (g.K + 31) >> 5;   // this workgroup's chunks: [s_begin, nlive)
  if (SLICES && g.kslices > 1) {
    s_begin = kslice * g.slice_chunks < nlive ? kslice * g.slice_chunks : nlive;
    nlive = s_begin + g.slice_chunks < nlive ? s_begin + g.slice_chunks : nlive;
  }
  const int per = (nlive - s_begin + KSPLIT - 1) / KSPLIT;
  const int c_begin = s_begin + kw_ * per;
  const int c_end = c_begin + per < nlive ? c_begin + per : nlive;
  const int niter = SLICES ? (per > 0 ? (per + D - 1) / D : 1) : (per + D - 1) / D;
  int cur = c_begin;
  int tap = 0, ch = 0, r = 0, s = 0;
  if (MODE != WAVE_IDENT && MODE != WAVE_ROWS) {
    tap = (int)fastdiv((unsigned)cur, g.div_ct);
    ch = (cur - tap * (g.dw ? 1 : ctiles)) * 32;
    r = (int)fastdiv((unsigned)tap, g.div_kw);
    s = tap - r * g.KW;
  }
  // depthwise form: K has one chunk per tap, the 32 input channels of this workgroup's own output channels
  const int cp_k = g.dw ? 32 : g.Cp;       // channels of one tap in K
  const int ch_first = g.dw ? oc0 : 0;     // first input channel this workgroup reads

  const __amdgpu_buffer_rsrc_t rs_w = act_rsrc(wf);   // the packed filter is smaller than 2^31 bytes (checked by the host)
  unsigned wa[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) wa[i] = (unsigned)(oc0 / 32 + (i ^ Xi)) * (unsigned)(nch + 1) * 1024u + (unsigned)((lane ^ (Q << 3)) * 16);
  const int lconst = lgrp * 512;
  unsigned tapoff[TN];                     // per-lane byte offset (from xp) of the current filter tap's granule; kOutsideBuffer
                                           // for a tap outside the image: a buffer load past the end reads zeros
  bool need_tap = true;
#pragma unroll
  for (int j = 0; j < TN; ++j) tapoff[j] = kOutsideBuffer;

  // (COH) The accumulators start from the bias: the addend of a tile's first MFMA is the bias of its 32 output channels as the
  // accumulator holds them (element e of a lane: channel (e / 4) * 8 + (lane / 32) * 4 + e % 4 of the tile), so the
  // epilogue neither reads nor adds it.  A launch of its own keeps the older form -- one word per lane requested
  // behind the first operand batch, staged in LDS after the K loop, added in the epilogue: there the four 16-byte
  // requests per 32 channels in front of the first operand request cost more than the epilogue's additions.  After a K split one wavefront of each tile set brings it in (the one whose
  // register groups are not permuted, kw_ == 0); the sums of the others start from zero.  The four 16-byte loads per
  // 32 channels are the first requests of the tile and hit two addresses per wavefront each.
  v16i binit[TM];
  {
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < TM; ++i) binit[i] = zero16;
    if (COH && ep.bias && (KSPLIT == 1 || kw_ == 0)) {
      const int OC = g.OC;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int first = oc0 + i * 32 + q * 8 + lgrp * 4;
          int4 bv;
          if (ep.bias_vec && (OC & 3) == 0) {   // whole groups of four channels, 16-byte aligned
            const bool ok = first < OC;
            bv = *reinterpret_cast<const int4*>(ep.bias + (ok ? first : 0));
            bv = ok ? bv : zero4();
          } else {
            int b4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bool ok = first + e < OC;
              const int b = ep.bias[ok ? first + e : 0];
              b4[e] = ok ? b : 0;
            }
            bv = make_int4(b4[0], b4[1], b4[2], b4[3]);
          }
          binit[i][q * 4] = bv.x; binit[i][q * 4 + 1] = bv.y; binit[i][q * 4 + 2] = bv.z; binit[i][q * 4 + 3] = bv.w;
        }
    }
  }
  v16i acc[TM][TN];   // first written by the first MFMA of each tile, whose addend is the bias

  // one batch = D chunks of both operands, one SSA value (see k_conv_igemm)
  typedef int regs_t __attribute__((ext_vector_type(4 * (TM + TN) * D)));
  auto put = [](regs_t& R, int b, const int4 v) __attribute__((always_inline)) {
    R[b] = v.x; R[b + 1] = v.y; R[b + 2] = v.z; R[b + 3] = v.w;
  };
  uint32_t rp[NU];
  // COH: called once, between the filter requests and the activation requests of the first batch
  auto pass_gate = [&]() __attribute__((always_inline)) {
    if constexpr (COH) {
      gate_wait(gate, wave);
      CVM_SEQ_STAMP(1, tid);
    }
  };
  // a filter chunk of tile row i: from memory, or (a layer with a chain behind it) from the copy of the filter in LDS
  auto load_w = [&](const int i, const unsigned chunk_bytes) __attribute__((always_inline)) -> int4 {
    if constexpr (TAIL >= 0) return *reinterpret_cast<const int4*>(chain_lds->w + wa[i] + chunk_bytes);
    else return ld16_buf<false>(rs_w, wa[i], chunk_bytes);
  };
  auto fetch = [&](const bool gated) __attribute__((always_inline)) -> regs_t {
    regs_t R;
    if (MODE == WAVE_IDENT) {
      // One path, loads always in the same order (filter blocks, then pixel blocks; the chunks of a
      // block together): with alternative paths that issue them in different orders the compiler
      // no longer knows how many younger loads may stay outstanding and drains them all before
      // every MFMA group.  A chunk past the end multiplies the all-zero filter chunk with a valid
      // activation address.
      int ca[D], cb[D];
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const bool live = cur + d < c_end;
        ca[d] = live ? cur + d : nch;
        cb[d] = live ? cur + d : (c_begin < nlive ? c_begin : 0);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int d = 0; d < D; ++d) put(R, (d * (TM + TN) + i) * 4, load_w(i, (unsigned)ca[d] * 1024u));
      if (gated) pass_gate();
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int d = 0; d < D; ++d) {
          put(R, (d * (TM + TN) + TM + j) * 4, ld16_buf<COH>(rs_x, xoff[j], (unsigned)cb[d] * 1024u));
        }
      cur = cur + D < c_end ? cur + D : c_end;
      return R;
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const bool live = cur < c_end;
      // a chunk past the end multiplies the all-zero filter chunk with a valid activation address
      const int chunk = live ? cur : nch;
#pragma unroll
      for (int i = 0; i < TM; ++i) put(R, (d * (TM + TN) + i) * 4, load_w(i, (unsigned)chunk * 1024u));
      if (gated && d == 0) pass_gate();
      if (MODE == WAVE_ROWS) {
        // 16-byte unit k16 of K: filter row k16 / (row_bytes/16), part k16 % (row_bytes/16) of its window
        const int k16 = (live ? cur : 0) * 2 + lgrp;
        const int sh16 = g.row_bytes >> 5;   // 0 or 1
        const int off = (k16 >> sh16) * (g.W * 4) + (k16 & sh16) * 16;
#pragma unroll
        for (int j = 0; j < TN; ++j) put(R, (d * (TM + TN) + TM + j) * 4, *reinterpret_cast<const int4*>(xp + (rowbase[j] + off)));
      } else {
        // the address of a pixel is computed once per filter tap; the Cp/32 chunks of
        // the tap differ by a multiple of 1 KiB (not applied to lanes that read zeros)
        if (live && need_tap) {
          const int soff = (r * g.DH) * g.W + s * g.DW;  // in pixels
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int pin = rowbase[j] + soff;
            const bool ok = MODE != WAVE_PAD || ((((rowmask[j] >> r) & (colmask[j] >> s)) & 1u) != 0);
            // Byte offset of the pixel's granule: block (pin / 32) * Cp * 32 + row (pin % 32) * 16.  The tensor
            // is smaller than 2^31 bytes (checked by the host), so a 24-bit multiply (full rate) is exact; for a
            // tap outside the image the offset is meaningless and the select below discards it -- a select, not
            // a branch, so that the two pointers cost a dozen instructions per tap instead of fifty.
            const unsigned off = __umul24((unsigned)pin >> 5, (unsigned)g.Cp << 5) + (((unsigned)pin & 31u) << 4) + (unsigned)lconst;
            tapoff[j] = ok ? off : kOutsideBuffer;
          }
          need_tap = false;
        }
        const int coff = live ? ((ch + ch_first) >> 5) * 1024 : 0;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          put(R, (d * (TM + TN) + TM + j) * 4, ld16_buf<COH>(rs_x, tapoff[j], (unsigned)coff));
        }
      }
      if (live) {
        ++cur;
        if (MODE != WAVE_ROWS) {
          ch += 32;
          if (ch >= cp_k) {
            ch = 0;
            ++tap;
            if (++s == g.KW) { s = 0; ++r; }
            need_tap = true;
          }
        }
      }
    }
    return R;
  };
  auto consume = [&](const regs_t R, const bool first) __attribute__((always_inline)) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      v4i a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int o = (d * (TM + TN) + i) * 4;
        a[i] = v4i{R[o], R[o + 1], R[o + 2], R[o + 3]};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int o = (d * (TM + TN) + TM + j) * 4;
        b[j] = v4i{R[o], R[o + 1], R[o + 2], R[o + 3]};
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], (first && d == 0) ? binit[i] : acc[i][j], 0, 0, 0);
    }
  };

  // Order of the requests: the residual of the groups this wavefront will finalise (nothing waits for
  // it before the epilogue; requested after the operands, its predicated form makes the compiler drain
  // every outstanding load first), the operands of the first batch, then the bias, which is kept in a
  // register and staged in LDS after the loop (staging it here would put a full memory latency in
  // front of the first operand request).
  if (!COH && ep.residual) load_residual<TN, NU, COH>(rp, kw_ * NU, 0, oc0, px0 + pw_ * TN * 32, lane, g, ep);
  regs_t R0 = fetch(COH);
  int bias_mine = 0;   // (!COH) this lane's word of the bias: without a K split every wavefront stages a copy of its own
  const int bias_lane = KSPLIT == 1 ? lane : tid;
  int* bias_lds = KSPLIT == 1 ? sBias + wave * BM : sBias;
  if constexpr (!COH) {
    if (bias_lane < BM) bias_mine = (ep.bias && oc0 + bias_lane < g.OC) ? ep.bias[oc0 + bias_lane] : 0;
  }
  // (Without a K split no wavefront needs anything from another one and the tile has no barrier at all: the
  // wavefronts of a workgroup drift apart, and one's epilogue runs under another's operand requests.)

  // (COH) the residual is not needed before the epilogue: requested behind the operand batches that are in flight
  // at the start, it does not stand between the layer boundary and the first MFMA
  auto residual_coh = [&]() __attribute__((always_inline)) {
    if constexpr (COH) {
      if (ep.residual) load_residual<TN, NU, COH>(rp, kw_ * NU, 0, oc0, px0 + pw_ * TN * 32, lane, g, ep);
    }
  };
  if (niter <= 1) {
    // the whole K range is one batch (a 1x1 layer over 64 channels): no second request.  Every byte a
    // wavefront asks for, used or not, takes its turn in the CU's memory pipeline, and these layers are
    // bound by exactly that.
    residual_coh();
    consume(R0, true);
    CVM_SEQ_STAMP(2, acc[0][0][0]);
  } else {
    regs_t R1 = fetch(false);
    residual_coh();
    consume(R0, true);
    CVM_SEQ_STAMP(2, acc[0][0][0]);
    for (int it = 1; it < niter; it += 2) {
      R0 = fetch(false);
      consume(R1, false);
      if (it + 1 >= niter) break;
      R1 = fetch(false);
      consume(R0, false);
    }
  }
  CVM_SEQ_STAMP(3, acc[0][0][0]);
  if constexpr (!COH) {
    if (bias_lane < BM) bias_lds[bias_lane] = bias_mine;
  }
  if constexpr (TAIL >= 0) {
    static_assert(TAIL < 0 || (KSPLIT == 1 && TN == 1 && COH && OUT == OUT_I8_ACT), "a chain starts from an unsplit tile of one pixel block");
    conv_chain_tail<TM, TAIL>(acc, ep, out, *tailB, tailC, *chain_lds, px0 + pw_ * 32, lane, p_begin, p_end);
    CVM_SEQ_STAMP(5, tid);
    return;
  }

  // ---- partial sums of the KSPLIT wavefronts that share a tile meet in LDS;
  // wavefront kw_ then finalises the groups kw_*NU .. kw_*NU + NU-1 of the tile set
  int32_t val[NU * 4];
  if (KSPLIT > 1) {
    int* mine = sPart + wave * U * 256;
#pragma unroll
    for (int u = NU; u < U; ++u) {   // the other wavefronts' groups
      const int t = u >> 2, q = u & 3;
      *reinterpret_cast<int4*>(mine + ((u ^ G) * 64 + lane) * 4) =
          make_int4(acc[t / TN][t % TN][q * 4], acc[t / TN][t % TN][q * 4 + 1], acc[t / TN][t % TN][q * 4 + 2],
                    acc[t / TN][t % TN][q * 4 + 3]);
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < NU; ++m) {   // own register group m = workgroup group G + m
      const int t = m >> 2, q = m & 3;
      int4 sum = make_int4(acc[t / TN][t % TN][q * 4], acc[t / TN][t % TN][q * 4 + 1], acc[t / TN][t % TN][q * 4 + 2],
                           acc[t / TN][t % TN][q * 4 + 3]);
#pragma unroll
      for (int d = 1; d < KSPLIT; ++d) {
        const int k = (kw_ + d) % KSPLIT;
        const int4 v = *reinterpret_cast<const int4*>(sPart + (((pw_ * KSPLIT + k) * U + G + m) * 64 + lane) * 4);
        sum.x = wadd(sum.x, v.x); sum.y = wadd(sum.y, v.y); sum.z = wadd(sum.z, v.z); sum.w = wadd(sum.w, v.w);
      }
      val[m * 4] = sum.x; val[m * 4 + 1] = sum.y; val[m * 4 + 2] = sum.z; val[m * 4 + 3] = sum.w;
    }
  } else {
    if constexpr (!COH) __builtin_amdgcn_wave_barrier();   // bias staged: written and read by this wavefront only, and LDS serves a wavefront in order
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) val[((i * TN + j) * 16 + e) % (NU * 4)] = acc[i][j][e];
  }
  CVM_SEQ_STAMP(4, val[0]);
  void* dst = out;
  if (SLICES && g.kslices > 1) dst = reinterpret_cast<int32_t*>(out) + (int64_t)kslice * g.slice_stride;   // int32 output only (host)
  finish_groups<TN, NU, OUT, COH, POOLR, COH, COH>(val, kw_ * NU, COH ? nullptr : bias_lds, 0, oc0, px0 + pw_ * TN * 32, lane, dst, g, ep, rp, p_begin, p_end);
  CVM_SEQ_STAMP(5, tid);
}

template <int TM, int TN, int KSPLIT, int NW, int D, int MINW, int OUT, int MODE, bool SLICES = false, bool POOLR = false>
__global__ void __launch_bounds__(NW * 64, MINW)
k_conv_wave(const int8_t* __restrict__ xp, const int8_t* __restrict__ wf, void* __restrict__ out,
            const ConvGeom g, const Epilogue ep) {
  constexpr int U = TM * TN * 4;
  __shared__ __attribute__((aligned(16))) int sPart[KSPLIT > 1 ? NW * U * 256 : 4];  // [wave][group][lane][4]
  __shared__ __attribute__((aligned(16))) int sBias[32 * TM * (KSPLIT == 1 ? NW : 1)];
  const int pid = xcd_tile_order(blockIdx.x, gridDim.x);
  conv_wave_tile<TM, TN, KSPLIT, NW, D, OUT, MODE, SLICES, false, POOLR>(xp, wf, out, g, ep, pid, threadIdx.x, sPart, sBias);
}

// ---------------------------------------------------------------- large-tile kernel
// Layers with enough output to fill the chip several times over (the 3x3 layers of a VGG) are bound by how
// many operand bytes an MFMA needs, not by latency.  Here a workgroup of four wavefronts, one per SIMD,
// owns a tile of up to 256 output channels x 256 pixels; each wavefront keeps a TM x TN block of 32x32
// MFMA tiles (4x4: 256 accumulator registers), so the 8 fragments it reads from LDS per 32 bytes of K
// feed 16 MFMAs.  Both operands reach LDS without passing through registers: global_load_lds_dwordx4
// takes one global address per lane and writes lane l's 16 bytes to (LDS base + 16 l), which is exactly the
// fragment order, so a wavefront gathers one 1 KiB fragment of the im2col matrix (padding taps read the
// zero granule) or of the packed filter per instruction.  K advances 64 bytes per step through a ring of
// NST stage buffers; a step is: wait until this wavefront's requests for the step have landed, one
// s_barrier, request the step NST-1 ahead into the buffer everyone has just left, then 2 x (TM + TN)
// ds_read_b128 and 2 x TM x TN MFMAs.  The barrier is the bare instruction and the waits are written by
// hand: the fence that comes with __syncthreads would wait for every outstanding request, i.e. undo the ring.
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int I, int TM, int TN, int OUT, bool POOLR>
__device__ __forceinline__ void big_epilogue_rows(v16i (&acc)[TM][TN], const int* sBias, int ch_wave, int oc0, int px_wave, int lane,
                                                  void* out, const ConvGeom& g, const Epilogue& ep) {
  if constexpr (I < TM) {
    int32_t val[TN * 16];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) val[j * 16 + e] = acc[I][j][e];
    uint32_t rp[TN * 4];
    if (ep.residual) load_residual<TN, TN * 4>(rp, I * TN * 4, ch_wave, oc0, px_wave, lane, g, ep);
    finish_groups<TN, TN * 4, OUT, false, POOLR>(val, I * TN * 4, sBias, ch_wave, oc0, px_wave, lane, out, g, ep, rp);
    big_epilogue_rows<I + 1, TM, TN, OUT, POOLR>(acc, sBias, ch_wave, oc0, px_wave, lane, out, g, ep);
  }
}

template <int WGM, int WGN, int TM, int TN, int OUT, bool POOLR = false>
__global__ void __launch_bounds__(256, (TM * TN <= 8 ? 2 : 1))
k_conv_big(const int8_t* __restrict__ xp, const int8_t* __restrict__ wf, void* __restrict__ out, const ConvGeom g, const Epilogue ep) {
  static_assert(WGM * WGN == 4, "four wavefronts");
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int NA = BM / 32, NB = BN / 32;               // 32-row blocks of the two operands
  constexpr int AF = NA * 2, BF = NB * 2;                  // fragments per stage (two 32-byte chunks of K)
  constexpr int STAGE = (AF + BF) * 1024;
  constexpr int NST = TM * TN <= 8 ? 3 : (STAGE * 4 <= 147456 ? 4 : 3);   // two workgroups per CU share the LDS when the tile is small
  constexpr int LA = AF / 4, LB = BF / 4;                  // requests per wavefront and stage
  constexpr int LPW = LA + LB;
  constexpr int PXW = NB / 4;                              // pixel blocks whose rows a wavefront gathers
  static_assert(NB % 4 == 0 && AF % 4 == 0, "pixel blocks and filter fragments are dealt to the four wavefronts");
  __shared__ __attribute__((aligned(16))) int8_t smem[NST * STAGE];
  __shared__ __attribute__((aligned(16))) int sBias[BM];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int pid = xcd_tile_order(blockIdx.x, gridDim.x);
  const int ptile = (int)fastdiv((unsigned)pid, g.div_octiles);
  const int oc0 = (pid - ptile * g.octiles) * BM;
  const int px0 = ptile * BN;
  const int P = (int)g.P;
  const int ctiles = g.Cp >> 5;
  const int nch = g.Kp >> 5, nlive = (g.K + 31) >> 5;
  const int nsteps = g.Kp >> 6;
  const int last_ot = ((g.OC + 127) / 128) * 4 - 1;       // last 32-row block the packed filter holds

  // ---- what this lane gathers: row (lane & 31) of PXW pixel blocks, bytes (lane >> 5) * 16 .. +15 of a chunk
  int rowbase[PXW];
  unsigned rowmask[PXW], colmask[PXW];
#pragma unroll
  for (int q = 0; q < PXW; ++q) {
    const int p = px0 + (wave + 4 * q) * 32 + lrow;
    const bool ok = p < P;
    const unsigned pp = ok ? (unsigned)p : 0u;
    int n, oh, ow;
    conv_out_pixel(g, ep.pool, pp, n, oh, ow);
    const int ih0 = oh * g.SH - g.PH, iw0 = ow * g.SW - g.PW;
    rowbase[q] = (n * g.H + ih0) * g.W + iw0;
    unsigned rm, cm;
    if (g.DH == 1 && g.DW == 1) {
      rm = tap_mask_dense(ih0, g.H, g.KH);
      cm = tap_mask_dense(iw0, g.W, g.KW);
    } else {
      rm = tap_mask_dilated(ih0, g.H, g.KH, g.DH);
      cm = tap_mask_dilated(iw0, g.W, g.KW, g.DW);
    }
    rowmask[q] = ok ? rm : 0u;
    colmask[q] = cm;
  }
  const int8_t* zero = reinterpret_cast<const int8_t*>(g_zero_granule);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lptr_t)smem;   // LDS byte address of the ring

  // ---- the request stream.  Stages are requested in order (the first NST - 1 before the loop, then one per step), so
  // the position in K is kept as running state instead of being decoded per request: chunk, its channel block and
  // filter tap (uniform), and per lane the address of the tap's granule for each pixel it gathers plus what one
  // channel block adds to it -- 1 KiB inside the image, nothing for a padding tap, whose address is the zero granule.
  // A request then costs one multiply-add per pixel; the address of a tap is worked out once per tap.  Requests past
  // the end of K (the ring runs NST - 1 stages ahead) read the zero granule and the slack behind the filter.
  int rq_cblk = 0, rq_r = 0, rq_s = 0, rq_tap = 0;
  uint64_t tap_addr[PXW];
  uint32_t tap_inc[PXW];
  uint64_t flt_addr[LA];      // this lane's 16 bytes of the filter fragments the wavefront requests, at the current step
#pragma unroll
  for (int t = 0; t < LA; ++t) {
    const int a = wave + 4 * t;                    // fragment (block a >> 1, chunk a & 1) of the filter
    int ot = (oc0 >> 5) + (a >> 1);
    ot = ot < last_ot ? ot : last_ot;              // blocks past the filter repeat its last one; their channels are never stored
    flt_addr[t] = (uint64_t)(uintptr_t)wf + ((uint64_t)ot * (nch + 1) + (a & 1)) * 1024 + lane * 16;
  }
  // One stage is LPW requests: `prepare` works out their addresses and advances the stream, `issue(i)` sends the
  // i-th.  They are sent one at a time between groups of MFMAs: a wavefront that sends a request is held until
  // the CU's address unit has taken all 64 lanes of it (1 KiB at 64 bytes a clock, behind the requests of the
  // other wavefronts), and eight of them back to back kept the MFMA pipes idle for longer than the MFMAs of a
  // stage take.
  uint64_t rq_addr[LPW];
  uint32_t rq_lds[LPW];
  auto prepare_filter = [&](int slot) __attribute__((always_inline)) {
    const uint32_t stage = lds_base + (uint32_t)(slot * STAGE);
#pragma unroll
    for (int t = 0; t < LA; ++t) {
      const int a = wave + 4 * t;
      rq_addr[t] = flt_addr[t];
      rq_lds[t] = stage + (uint32_t)a * 1024u;
      flt_addr[t] += 2048;
    }
  };
  auto prepare_chunk = [&](int slot, int c) __attribute__((always_inline)) {
    const uint32_t stage = lds_base + (uint32_t)(slot * STAGE);
    {
      if (rq_cblk == 0) {       // a new tap (uniform, once per Cp / 32 chunks)
        const bool tap_ok = rq_tap < g.taps;
        const int soff = (rq_r * g.DH) * g.W + rq_s * g.DW;
#pragma unroll
        for (int q = 0; q < PXW; ++q) {
          const int pin = rowbase[q] + soff;
          const bool ok = tap_ok && ((((rowmask[q] >> rq_r) & (colmask[q] >> rq_s)) & 1u) != 0);
          const unsigned off = __umul24((unsigned)pin >> 5, (unsigned)g.Cp << 5) + (((unsigned)pin & 31u) << 4) + (unsigned)(lgrp * 512);
          const uint64_t inside = (uint64_t)(uintptr_t)xp + off, outside = (uint64_t)(uintptr_t)zero;
          tap_addr[q] = outside ^ ((inside ^ outside) & (ok ? ~0ull : 0ull));
          tap_inc[q] = ok ? 1024u : 0u;
        }
      }
#pragma unroll
      for (int q = 0; q < PXW; ++q) {
        rq_addr[LA + c * PXW + q] = tap_addr[q];
        tap_addr[q] += tap_inc[q];             // the next channel block of the tap
        rq_lds[LA + c * PXW + q] = stage + (uint32_t)(AF + (wave + 4 * q) * 2 + c) * 1024u;
      }
      if (++rq_cblk == ctiles) {
        rq_cblk = 0;
        ++rq_tap;
        if (++rq_s == g.KW) { rq_s = 0; ++rq_r; }
      }
    }
  };
  auto prepare = [&](int slot) __attribute__((always_inline)) {
    prepare_filter(slot);
    prepare_chunk(slot, 0);
    prepare_chunk(slot, 1);
  };
  auto issue = [&](int i) __attribute__((always_inline)) {
    lds_dma16(reinterpret_cast<const void*>((uintptr_t)rq_addr[i]), rq_lds[i]);
  };

  v16i acc[TM][TN];
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = zero16;

  // ---- the ring.  A step multiplies the fragments of its first chunk while those of its second chunk are read from
  // LDS, then meets the other wavefronts once (its own requests for the next step have landed, it has read the last
  // fragment of this step's slot), and multiplies the second chunk while the first chunk of the next step is read.
  // The slot just left is refilled with the step NST ahead: H1 of its requests go out during this step's second
  // half, the other H2 during the next step's first half.  Everything that is not an MFMA -- an LDS read, a
  // request, a piece of the address arithmetic -- is placed behind one particular MFMA, a few instructions at a
  // time: a wavefront issues in order, an MFMA keeps the matrix pipe busy for 32 clocks, and only what is issued
  // inside those 32 clocks is free.  (In blocks between groups of MFMAs the same instructions left the pipe idle
  // for half of a step when the workgroup had the CU to itself.)
  constexpr int H1 = LPW / 2, H2 = LPW - H1, NM = TM * TN;
  static_assert(H2 <= NM - 3 && TM + TN <= NM, "a half step has an MFMA for every request, LDS read and piece of address arithmetic");
  auto lds16 = [&](const int8_t* p) __attribute__((always_inline)) { return *reinterpret_cast<const v4i*>(p + lane * 16); };
#pragma unroll
  for (int st = 0; st < NST; ++st) {
    prepare(st);
#pragma unroll
    for (int i = 0; i < (st < NST - 1 ? LPW : H1); ++i) issue(i);   // the last slot's other requests go out in the first step
  }
  stage_bias<BM>(sBias, ep, g.OC, oc0, tid);
  v4i a0[TM], b0[TN], a1[TM], b1[TN];
  wait_vm<(NST - 2) * LPW + H1>();
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int i = 0; i < TM; ++i) a0[i] = lds16(smem + ((wm * TM + i) * 2) * 1024);
#pragma unroll
  for (int j = 0; j < TN; ++j) b0[j] = lds16(smem + (AF + (wn * TN + j) * 2) * 1024);
  int slot = 0;
  for (int kt = 0; kt < nsteps; ++kt) {
    const int8_t* stage = smem + slot * STAGE;
    // first half: chunk 0; behind its MFMAs the reads of chunk 1, the H2 requests still owed to the slot refilled in
    // the previous step, and then the addresses of step kt + NST, which goes into the slot being left
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      acc[m / TN][m % TN] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0[m / TN], b0[m % TN], acc[m / TN][m % TN], 0, 0, 0);
      if (m < TM) a1[m] = lds16(stage + ((wm * TM + m) * 2 + 1) * 1024);
      else if (m < TM + TN) b1[m - TM] = lds16(stage + (AF + (wn * TN + (m - TM)) * 2 + 1) * 1024);
#pragma unroll
      for (int r = 0; r < H2; ++r)
        if (m == r * (NM - 3) / H2) issue(H1 + r);
      if (m == NM - 3) prepare_filter(slot);
      if (m == NM - 2) prepare_chunk(slot, 0);
      if (m == NM - 1) prepare_chunk(slot, 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot has been read completely
    wait_vm<(NST - 2) * LPW>();                             // own requests of the next step have landed
    __builtin_amdgcn_s_barrier();
    const int next = slot + 1 == NST ? 0 : slot + 1;
    const int8_t* nstage = smem + next * STAGE;
    // second half: chunk 1; behind its MFMAs the reads of the next step's chunk 0 and the first H1 requests of the refill
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      acc[m / TN][m % TN] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1[m / TN], b1[m % TN], acc[m / TN][m % TN], 0, 0, 0);
      if (m < TM) a0[m] = lds16(nstage + ((wm * TM + m) * 2) * 1024);
      else if (m < TM + TN) b0[m - TM] = lds16(nstage + (AF + (wn * TN + (m - TM)) * 2) * 1024);
#pragma unroll
      for (int r = 0; r < H1; ++r)
        if (m == r * NM / H1) issue(r);
      __builtin_amdgcn_sched_barrier(0);
    }
    slot = next;
  }
  wait_vm<0>();      // the requests that ran past the end of K
  __syncthreads();   // bias staged (all requests have landed by now)

  // ---- epilogue, one row of TN tiles at a time (the row index is a template argument: an accumulator indexed by a
  // loop variable that the compiler does not unroll would be moved to scratch memory as a whole)
  big_epilogue_rows<0, TM, TN, OUT, POOLR>(acc, sBias, wm * TM * 32, oc0, px0 + wn * TN * 32, lane, out, g, ep);
}

// ---------------------------------------------------------------- row-window convolution + 3x3 stride-2 max-pool
// The head of a ResNet: a convolution over a few input channels (row-window form, see StemGeom) whose only reader
// is max_pool2d with a 3x3 window, stride 2 and padding 1 (ops.cc:466-523).  A workgroup computes a patch of
// 4 x 8 pooled pixels of one image for up to 64 output channels: the 9 x 17 convolution pixels under it (windows
// overlap, so neighbouring patches share a row and a column: 1.2 x the multiply-adds, which are a small part of a
// launch that is all latency) go through the requantisation chain into LDS as int8, pixels outside the
// convolution's output as -128 (every window holds at least one real pixel, so the padding never wins), and a
// second phase takes the maxima.  The convolution's output never reaches memory and the pool's launch goes away.
// A workgroup's chain of steps is long (0.6 us of addresses, 2 us of requests and MFMAs, 1.8 us of requantisation
// into LDS, 0.6 us of maxima at one workgroup per CU), so this pays while the grid is a single round of workgroups
// (a ResNet's head at batch 1: 8.0 against 4.0 + 4.7 us and a launch gap); at batch 16 its three rounds take 22 us
// against 17 us for the two launches, and the caller keeps those.
struct StemPool {
  int N, Hs, Ws;         // stored (zero padded) input extent in pixels of 4 bytes
  int OH, OW, QH, QW;    // extent of the convolution's and of the pool's output
  int SH, SW, OC, ocp;
  int nch, nlive, sh16;  // chunks per row of the packed filter (zero chunk at nch), chunks of the true K, row_bytes >> 5
  int tiles_x, tiles_y;
  DevChain chain;
  const int32_t* bias;
};
constexpr int SP_PH = 4, SP_PW = 8, SP_CH = 2 * SP_PH + 1, SP_CW = 2 * SP_PW + 1, SP_PIX = SP_CH * SP_CW;
constexpr int SP_BLOCKS = (SP_PIX + 31) / 32, SP_SLOTS = (SP_BLOCKS + 1) / 2, SP_BATCH = 8;

__global__ void __launch_bounds__(256, 2)
k_stem_pool(const int8_t* __restrict__ xs, const int8_t* __restrict__ wf, int8_t* __restrict__ out, const StemPool a) {
  __shared__ __attribute__((aligned(16))) int8_t sTile[SP_BLOCKS * 32 * 64];   // [convolution pixel of the patch][64 channels]
  __shared__ int sBias[64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lgrp = lane >> 5;
  const int tx = blockIdx.x, ty = blockIdx.y, n = blockIdx.z;
  const int cy0 = 2 * ty * SP_PH - 1, cx0 = 2 * tx * SP_PW - 1;   // first convolution row / column of the patch
  if (tid < 64) sBias[tid] = (a.bias && tid < a.OC) ? a.bias[tid] : 0;
  // wavefront: channel tile (wave & 1), pixel blocks (wave >> 1), + 2, + 4
  const int ot = wave & 1, bg = wave >> 1;
  const bool has_tile = ot * 32 < a.OC;   // uniform
  unsigned rowbase[SP_SLOTS];
  bool inside[SP_SLOTS];
#pragma unroll
  for (int j = 0; j < SP_SLOTS; ++j) {
    int p = (bg + 2 * j) * 32 + lrow;
    const bool in_patch = p < SP_PIX;
    p = in_patch ? p : SP_PIX - 1;
    const int py = p / SP_CW, px = p - py * SP_CW;
    const int oh = cy0 + py, ow = cx0 + px;
    inside[j] = in_patch && oh >= 0 && oh < a.OH && ow >= 0 && ow < a.OW;
    const int ohc = oh < 0 ? 0 : (oh > a.OH - 1 ? a.OH - 1 : oh), owc = ow < 0 ? 0 : (ow > a.OW - 1 ? a.OW - 1 : ow);
    rowbase[j] = (unsigned)(((n * a.Hs + ohc * a.SH) * a.Ws + owc * a.SW) * 4);   // a pixel outside computes a neighbour's value, unused
  }
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  v16i acc[SP_SLOTS];
#pragma unroll
  for (int j = 0; j < SP_SLOTS; ++j) acc[j] = zero16;
  if (has_tile) {
    // all chunks of a 7-row filter are requested before the first is used: one trip to memory instead of two
    for (int c0 = 0; c0 < a.nlive; c0 += SP_BATCH) {
      v4i f[SP_BATCH], x[SP_BATCH][SP_SLOTS];
#pragma unroll
      for (int d = 0; d < SP_BATCH; ++d) {
        const int c = c0 + d;
        const bool live = c < a.nlive;   // a chunk past the end multiplies the filter's all-zero chunk
        f[d] = *reinterpret_cast<const v4i*>(wf + ((size_t)(ot * (a.nch + 1) + (live ? c : a.nch)) * 1024 + lane * 16));
        // 16-byte unit k16 of K: filter row k16 >> sh16, part k16 & sh16 of its window
        const int k16 = (live ? c : 0) * 2 + lgrp;
        const unsigned off = (unsigned)((k16 >> a.sh16) * (a.Ws * 4) + (k16 & a.sh16) * 16);
#pragma unroll
        for (int j = 0; j < SP_SLOTS; ++j)
          if (bg + 2 * j < SP_BLOCKS) x[d][j] = *reinterpret_cast<const v4i*>(xs + rowbase[j] + off);
      }
#pragma unroll
      for (int d = 0; d < SP_BATCH; ++d)
#pragma unroll
        for (int j = 0; j < SP_SLOTS; ++j)
          if (bg + 2 * j < SP_BLOCKS) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f[d], x[d][j], acc[j], 0, 0, 0);
    }
  }
  __syncthreads();   // bias staged
  if (has_tile) {
#pragma unroll
    for (int j = 0; j < SP_SLOTS; ++j) {
      if (bg + 2 * j >= SP_BLOCKS) continue;
      int32_t val[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int4 bv = *reinterpret_cast<const int4*>(sBias + ot * 32 + q * 8 + lgrp * 4);
        val[q * 4] = wadd(acc[j][q * 4], bv.x); val[q * 4 + 1] = wadd(acc[j][q * 4 + 1], bv.y);
        val[q * 4 + 2] = wadd(acc[j][q * 4 + 2], bv.z); val[q * 4 + 3] = wadd(acc[j][q * 4 + 3], bv.w);
      }
      run_chain(a.chain, val);
      const int p = (bg + 2 * j) * 32 + lrow;   // < SP_BLOCKS * 32: inside sTile
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t pk = inside[j] ? pack_bytes(val[q * 4], val[q * 4 + 1], val[q * 4 + 2], val[q * 4 + 3]) : 0x80808080u;
        *reinterpret_cast<uint32_t*>(sTile + p * 64 + ot * 32 + q * 8 + lgrp * 4) = pk;
      }
    }
  }
  __syncthreads();
  // ---- the maxima: one thread per pooled pixel and 16 channels
  if (tid < SP_PH * SP_PW * 4) {
    const int g16 = tid & 3, q = tid >> 2;
    const int qy = q / SP_PW, qx = q - qy * SP_PW;
    const int QY = ty * SP_PH + qy, QX = tx * SP_PW + qx;
    if (QY < a.QH && QX < a.QW && g16 * 16 < a.ocp) {
      int4 v[9];
#pragma unroll
      for (int dy = 0; dy < 3; ++dy)
#pragma unroll
        for (int dx = 0; dx < 3; ++dx)
          v[dy * 3 + dx] = *reinterpret_cast<const int4*>(sTile + ((2 * qy + dy) * SP_CW + 2 * qx + dx) * 64 + g16 * 16);
      const int4 m = max_pool_reduce<9>(v);
      *reinterpret_cast<int4*>(out + act_offset((int64_t)(n * a.QH + QY) * a.QW + QX, g16 * 16, a.ocp)) = m;
    }
  }
}

// ---------------------------------------------------------------- layer-sequence kernel
// A run of convolutions of one graph in ONE launch.  The images are dealt to 8, 4, 2 or 1 of the chip's 8 XCDs (the
// largest of these that divides the batch; workgroups on the other XCDs leave at once).
// Images are independent, so XCD x computes every layer for its own share of the images (pixel range
// [x * px_per_share, (x + 1) * px_per_share) of every tensor) and never reads what another XCD wrote.  The
// 32 compute units of an XCD share one L2, which makes a layer boundary cheap and local:
//   * a producer's ordinary stores are in the L2 once its wavefronts have waited for them (vmcnt);
//   * the consumers read activations and residuals with device-scope loads (ld16_l2), which the L2 answers;
//   * the boundary itself is one counter per XCD in that L2 (an atomic add per workgroup, then polling) --
//     no L2 write-back or invalidation, which is what makes a kernel boundary or an agent-scope
//     release cost microseconds; the dirty lines leave the L2 when the kernel ends, as after any kernel.
// One workgroup of 8 wavefronts per compute unit (grid = 256); it learns its XCD from the hardware
// register, its rank among the workgroups of that XCD from the order of arrival, and walks the tiles
// rank, rank + 32, ... of every layer (configurations of 4 wavefronts run two tiles side by side).
// Every wait is bounded: when a counter does not arrive within spin_limit polls the workgroup raises
// the error flag, which makes every workgroup leave at its next boundary; the host then falls back to one
// launch per layer.
// A step between two boundaries is one layer, or a layer with the 1x1 layers chained behind it (SeqLayer::chain), or
// two layers that have nothing to do with one another (SeqLayer::join_next); conv_seq_link decides on the host.
template <int TM, int TN, int KSPLIT, int NW, int D, int MODE>
__device__ __forceinline__ void seq_layer_tiles(const int8_t* xp, const int8_t* wf, void* out, const ConvGeom& g, const Epilogue& ep,
                                                int ntiles, int dead_tile, int rank, int tid, int* sPart, int* sBias, int p_begin,
                                                int p_end, const LayerGate gate, unsigned long long* tr) {
  constexpr int UNITS = 8 / NW;   // tiles a workgroup computes side by side
  const int half = UNITS == 2 ? (tid >> 8) : 0;
  const int htid = UNITS == 2 ? (tid & 255) : tid;
  for (int base = 0; base < ntiles; base += SEQ_WG_PER_SHARE * UNITS) {
    const int t = base + half * SEQ_WG_PER_SHARE + rank;   // the first 32 tiles go to 32 different compute units
    conv_wave_tile<TM, TN, KSPLIT, NW, D, OUT_I8_ACT, MODE, false, true>(
        xp, wf, out, g, ep, t < ntiles ? t : dead_tile, htid, sPart + half * 16384, sBias + half * 256, p_begin, p_end,
        base == 0 ? LayerGate{gate.counter, gate.target, gate.error, gate.spin_limit, gate.seen + half} : LayerGate{nullptr, 0, nullptr, 0, nullptr},
        base == 0 ? tr : nullptr);
    if (KSPLIT > 1) __syncthreads();   // the next tile reuses the LDS of the partial sums
  }
}

template <int MODE>
__device__ __forceinline__ void seq_layer_cfg(int cfg, const int8_t* xp, const int8_t* wf, void* out, const ConvGeom& g, const Epilogue& ep,
                                              int ntiles, int dead_tile, int rank, int tid, int* sPart, int* sBias, int p_begin,
                                              int p_end, const LayerGate gate, unsigned long long* tr) {
  switch (cfg) {
    case 0: seq_layer_tiles<2, 2, 8, 8, 2, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    case 1: seq_layer_tiles<2, 2, 4, 4, 2, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    case 2: seq_layer_tiles<2, 2, 2, 4, 2, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    case 3: seq_layer_tiles<2, 2, 1, 4, 2, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    case 4: seq_layer_tiles<1, 2, 8, 8, 4, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    case 5: seq_layer_tiles<1, 2, 4, 4, 4, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
    default: seq_layer_tiles<1, 2, 1, 4, 4, MODE>(xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr); break;
  }
}

// A layer with a chain behind it: 64 output channels x 32 pixels per wavefront, unsplit.  Every wavefront is a tile of its
// own, pixel block `wave * 32 + rank` of the share: up to 256 blocks run in one round, spread evenly over the 32
// workgroups.  Before the tiles the workgroup as a whole requests the chain's filters and biases into LDS, waits at the
// layer boundary (its first wavefront polls, the others watch its word in LDS) and meets at a barrier when the copies
// have landed; from there on no wavefront needs another.  mt1: 32-channel tiles of the chain's second layer (0: none).
template <int MODE, int TAIL>
__device__ __forceinline__ void seq_chain_tiles(const SeqLayer& A, int ntiles, int dead_tile, int rank, int tid, int* sPart, int* sBias,
                                                int p_begin, int p_end, const LayerGate gate, unsigned long long* tr,
                                                const SeqLayer* tailB, const SeqLayer* tailC) {
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const ChainLds lds = chain_stage_operands(A, *tailB, TAIL > 0 ? tailC : nullptr, sPart, sBias, tid);
  gate_wait(gate, wave);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const LayerGate none = {nullptr, 0, nullptr, 0, nullptr};
  for (int base = 0; base < ntiles; base += 8 * SEQ_WG_PER_SHARE) {
    const int t = base + wave * SEQ_WG_PER_SHARE + rank;
    if (t >= ntiles) continue;
    conv_wave_tile<2, 1, 1, 1, 4, OUT_I8_ACT, MODE, false, true, false, TAIL>(
        A.xp, A.wf, A.out, A.g, A.ep, t, tid & 63, sPart, sBias, p_begin, p_end, none, base == 0 && wave == 0 ? tr : nullptr, tailB, tailC, &lds);
  }
}
template <int MODE>
__device__ __forceinline__ void seq_layer_chain(int mt1, const SeqLayer& A, int ntiles, int dead_tile, int rank, int tid, int* sPart,
                                                int* sBias, int p_begin, int p_end, const LayerGate gate, unsigned long long* tr,
                                                const SeqLayer* tailB, const SeqLayer* tailC) {
  switch (mt1) {
    case 0: seq_chain_tiles<MODE, 0>(A, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC); break;
    case 2: seq_chain_tiles<MODE, 2>(A, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC); break;
    default: seq_chain_tiles<MODE, 4>(A, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC); break;
  }
}

__global__ void __launch_bounds__(512, 1)
k_conv_seq(const SeqLayer* __restrict__ layers_generic, int nlayers, unsigned* __restrict__ sync, int spin_limit,
           unsigned long long* __restrict__ stamps, int stamp_layers) {
  __shared__ __attribute__((aligned(16))) int sPart[32768];   // 128 KiB: one 8-wavefront tile set or two 4-wavefront ones
  __shared__ __attribute__((aligned(16))) int sBias[512];    // per half: one copy, or one per wavefront of an unsplit tile
  __shared__ int s_rank;
  __shared__ unsigned s_seen[2];   // per half of the workgroup: the highest layer boundary its first wavefront has seen reached
  // The table entries of the current layer (and of the one or two chained behind it) live in LDS, where any field is a
  // short read away wherever the code needs it (a copy in registers would hold ~100 scalar registers for the whole
  // layer, and reading it from memory would begin every layer with a trip there): a ring of eight slots, entry e in
  // slot e % 8.  When a step over `cnt` entries begins, entries l .. l + 2 are in the ring; the first wavefront requests
  // the entries l + 3 .. l + 2 + cnt, which arrive in their slots before the layer boundary.
  constexpr int LWORDS = (int)(sizeof(SeqLayer) / 4);
  constexpr int RING = 8;
  static_assert(sizeof(SeqLayer) % 16 == 0 && LWORDS <= 128, "a table entry is copied by one wavefront, two words per lane");
  __shared__ __attribute__((aligned(16))) uint32_t sLayer[RING][LWORDS];
  const uint32_t* table_words = reinterpret_cast<const uint32_t*>(layers_generic);
  for (int w = threadIdx.x; w < 3 * LWORDS; w += 512) {
    const int e = w / LWORDS;
    if (e < nlayers) sLayer[e][w - e * LWORDS] = table_words[w];
  }
  const int tid = threadIdx.x;
  unsigned xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  xcc &= 15u;
  __syncthreads();   // the first table entries are in LDS
  // a batch that does not divide over all 8 XCDs runs on the first `shares` of them; a workgroup elsewhere has nothing to do
  if (xcc < SEQ_SHARES && (int)xcc >= reinterpret_cast<const SeqLayer*>(sLayer[0])->shares) return;
  unsigned* my = sync + (xcc < SEQ_SHARES ? xcc : 0) * SEQ_SYNC_WORDS;
  unsigned* error = sync + SEQ_SHARES * SEQ_SYNC_WORDS;
  if (tid == 0) {
    const unsigned r = __hip_atomic_fetch_add(my + SEQ_ARRIVE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // not the chip this kernel is laid out for; or no patience at all, which is how a host tests its fall-back: the launch
    // then reports failure whatever happens, and no wait inside it ever sleeps
    if (xcc >= SEQ_SHARES || r >= SEQ_WG_PER_SHARE || spin_limit <= 0) __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_rank = (int)r;
    s_seen[0] = s_seen[1] = 0u;
  }
  __syncthreads();
  const int rank = s_rank;
  const bool stop = xcc >= SEQ_SHARES || rank >= SEQ_WG_PER_SHARE;
  int step = 0;          // layer boundaries passed: a chain of layers is one step, and so are two layers joined without a boundary
  bool joined = false;   // no boundary behind the previous layer: this one does not wait
  for (int l = 0; l < nlayers && !stop;) {
    const SeqLayer& L = *reinterpret_cast<const SeqLayer*>(sLayer[l & (RING - 1)]);
    const int chain = __builtin_amdgcn_readfirstlane(L.chain);
    const int cnt = chain + 1;   // table entries this step consumes (at most 3)
    // (memory -> LDS without passing through registers: held in registers for the length of a layer, the entries cost
    // every tile loop of the kernel, all of which use the whole register file, a spill)
    if (tid < LWORDS / 4) {
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const int e = l + 3 + k;
        if (k < cnt && e < nlayers)
          lds_dma16(table_words + (size_t)e * LWORDS + tid * 4,
                    (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(uintptr_t)(lptr_t)&sLayer[e & (RING - 1)][0]));
      }
    }
    const ConvGeom& g = L.g;
    const Epilogue& ep = L.ep;
    const int8_t* xp = L.xp;
    const int8_t* wf = L.wf;
    void* out = L.out;
    const int kernel = L.kernel;
    const int p_begin = (int)xcc * L.px_per_share;
    const int p_end = p_begin + L.px_per_share;
    const int ntiles = g.octiles * L.ptiles;
    const int dead_tile = g.octiles * (L.ptiles + 1);   // a tile past the share: computes, stores nothing
    const int cfg = kernel / 3, mode = kernel - cfg * 3;
    // this step may read what the previous one wrote once all 32 workgroups of the XCD have counted themselves out of it
    const LayerGate gate = {step > 0 && !joined ? my + SEQ_BAR : nullptr, (unsigned)step * SEQ_WG_PER_SHARE, error, spin_limit, s_seen};
#ifdef CVM_SEQ_STAMPS
    unsigned long long* tr = stamps && l < stamp_layers ? stamps + ((size_t)((int)xcc * SEQ_WG_PER_SHARE + rank) * stamp_layers + l) * 8 : nullptr;
    if (tr && tid == 0) tr[7] = __builtin_amdgcn_s_memtime();
#else
    unsigned long long* tr = nullptr;
#endif
    if (chain > 0) {
      const SeqLayer* tailB = reinterpret_cast<const SeqLayer*>(sLayer[(l + 1) & (RING - 1)]);
      const SeqLayer* tailC = reinterpret_cast<const SeqLayer*>(sLayer[(l + 2) & (RING - 1)]);
      const int mt1 = chain > 1 ? __builtin_amdgcn_readfirstlane(tailC->g.OC) >> 5 : 0;
      if (mode == 0) seq_layer_chain<WAVE_IDENT>(mt1, L, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC);
      else if (mode == 1) seq_layer_chain<WAVE_NOPAD>(mt1, L, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC);
      else seq_layer_chain<WAVE_PAD>(mt1, L, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr, tailB, tailC);
    } else if (mode == 0) seq_layer_cfg<WAVE_IDENT>(cfg, xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr);
    else if (mode == 1) seq_layer_cfg<WAVE_NOPAD>(cfg, xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr);
    else seq_layer_cfg<WAVE_PAD>(cfg, xp, wf, out, g, ep, ntiles, dead_tile, rank, tid, sPart, sBias, p_begin, p_end, gate, tr);
    if (l + cnt >= nlayers) {
#ifdef CVM_SEQ_STAMPS
      if (tr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) tr[6] = __builtin_amdgcn_s_memtime();
      }
#endif
      break;
    }
    joined = __builtin_amdgcn_readfirstlane(L.join_next) != 0;
    if (joined) {
      // no boundary: only the table entries requested at the layer's start must be in LDS before anyone looks for them
      if (tid < 64) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    } else {
      // ---- this workgroup is done with the step: every store of its wavefronts is in the L2 (and the table entries
      // requested at its start are in LDS), then it counts itself out
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) __hip_atomic_fetch_add(my + SEQ_BAR, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ++step;
    }
#ifdef CVM_SEQ_STAMPS
    if (tr && tid == 0) tr[6] = __builtin_amdgcn_s_memtime();
#endif
    l += cnt;
  }
  // the last workgroup of a share to finish clears the share's counters for the next launch
  __syncthreads();
  if (tid == 0 && xcc < SEQ_SHARES) {
    const unsigned d = __hip_atomic_fetch_add(my + SEQ_DONE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (d == SEQ_WG_PER_SHARE - 1) {
      __hip_atomic_store(my + SEQ_ARRIVE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(my + SEQ_BAR, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(my + SEQ_DONE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---------------------------------------------------------------- independent convolutions in one launch
// Convolutions with int32 output that do not depend on one another (the detection heads of a network: seven launches
// of 4 to 128 workgroups each, every one a chain of latencies on a mostly idle chip) as ONE grid.  The table gives
// layer k the workgroup indices [first_k, first_k + blocks_k); a workgroup looks its layer up, copies the entry to
// LDS and runs that layer's tile with the 8-wavefront configuration (64 or 32 output channels, K split 8 ways)
// the table names.  Entries are SeqLayer records; px_per_share holds first_k and ptiles holds blocks_k.
template <int MODE>
__device__ __forceinline__ void group_layer_cfg(int cfg, const int8_t* xp, const int8_t* wf, void* out, const ConvGeom& g,
                                                const Epilogue& ep, int pid, int tid, int* sPart, int* sBias) {
  if (cfg == 0) conv_wave_tile<2, 2, 8, 8, 2, OUT_I32_NCHW, MODE, false, false>(xp, wf, out, g, ep, pid, tid, sPart, sBias);
  else conv_wave_tile<1, 2, 8, 8, 4, OUT_I32_NCHW, MODE, false, false>(xp, wf, out, g, ep, pid, tid, sPart, sBias);
}

__global__ void __launch_bounds__(512, 1)
k_conv_group(const SeqLayer* __restrict__ layers, int nlayers) {
  __shared__ __attribute__((aligned(16))) int sPart[32768];   // 128 KiB: the partial sums of a 64 x 64 tile split 8 ways
  __shared__ __attribute__((aligned(16))) int sBias[64];
  constexpr int LWORDS = (int)(sizeof(SeqLayer) / 4);
  __shared__ __attribute__((aligned(16))) uint32_t sLayer[LWORDS];
  const int tid = threadIdx.x;
  const int bid = blockIdx.x;
  int l = 0;
  for (int k = 1; k < nlayers; ++k)
    if (bid >= layers[k].px_per_share) l = k;   // first workgroup index of layer k; ascending
  if (tid < LWORDS) sLayer[tid] = reinterpret_cast<const uint32_t*>(layers + l)[tid];
  __syncthreads();
  const SeqLayer& L = *reinterpret_cast<const SeqLayer*>(sLayer);
  const int pid = bid - L.px_per_share;
  const int cfg = L.kernel / 3, mode = L.kernel - cfg * 3;
  if (mode == 0) group_layer_cfg<WAVE_IDENT>(cfg, L.xp, L.wf, L.out, L.g, L.ep, pid, tid, sPart, sBias);
  else if (mode == 1) group_layer_cfg<WAVE_NOPAD>(cfg, L.xp, L.wf, L.out, L.g, L.ep, pid, tid, sPart, sBias);
  else group_layer_cfg<WAVE_PAD>(cfg, L.xp, L.wf, L.out, L.g, L.ep, pid, tid, sPart, sBias);
}

// The same for convolutions with int8 output (independent layers of a network at a small batch, e.g. the first 1x1 layer
// and the shortcut projection of a ResNet block, each far fewer workgroups than the chip has CUs): 32-channel tiles, K
// split 8 ways, 64 KiB of partial sums, so two workgroups share a CU.
// (a layer with fewer than two chunks of K per wavefront after an 8-way split runs unsplit instead: its eight
// wavefronts then take eight pixel tiles side by side)
template <int MODE>
__device__ __forceinline__ void group8_layer(const SeqLayer& L, int pid, int tid, int* sPart, int* sBias) {
  if (L.kernel / 3 == 4) conv_wave_tile<1, 2, 8, 8, 4, OUT_I8_ACT, MODE, false, false>(L.xp, L.wf, L.out, L.g, L.ep, pid, tid, sPart, sBias);
  else conv_wave_tile<1, 2, 1, 8, 4, OUT_I8_ACT, MODE, false, false>(L.xp, L.wf, L.out, L.g, L.ep, pid, tid, sPart, sBias);
}
__global__ void __launch_bounds__(512, 2)
k_conv_group8(const SeqLayer* __restrict__ layers, int nlayers) {
  __shared__ __attribute__((aligned(16))) int sPart[16384];
  __shared__ __attribute__((aligned(16))) int sBias[256];   // unsplit: a copy per wavefront
  constexpr int LWORDS = (int)(sizeof(SeqLayer) / 4);
  __shared__ __attribute__((aligned(16))) uint32_t sLayer[LWORDS];
  const int tid = threadIdx.x;
  const int bid = blockIdx.x;
  int l = 0;
  for (int k = 1; k < nlayers; ++k)
    if (bid >= layers[k].px_per_share) l = k;
  if (tid < LWORDS) sLayer[tid] = reinterpret_cast<const uint32_t*>(layers + l)[tid];
  __syncthreads();
  const SeqLayer& L = *reinterpret_cast<const SeqLayer*>(sLayer);
  const int pid = bid - L.px_per_share;
  const int mode = L.kernel % 3;
  if (mode == 0) group8_layer<WAVE_IDENT>(L, pid, tid, sPart, sBias);
  else if (mode == 1) group8_layer<WAVE_NOPAD>(L, pid, tid, sPart, sBias);
  else group8_layer<WAVE_PAD>(L, pid, tid, sPart, sBias);
}

// Second step of a K-sliced convolution: out = chain(sum over slices + bias), stored like the epilogue would
// (int8 activations or int32 NCHW).  One thread per 4 consecutive channels of a pixel.
template <int OUT>
__global__ void __launch_bounds__(256) k_slices_finish(const int32_t* __restrict__ part, void* __restrict__ out, int kslices,
                                                       int slice_stride, const ConvGeom g, const Epilogue ep) {
  const int OHW = g.OH * g.OW;
  const int oc4 = OUT == OUT_I8_ACT ? ep.out_cp >> 2 : (g.OC + 3) >> 2;   // int8: padding channels are written too (as zeros)
  const int64_t total = g.P * oc4;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t p = i / oc4;
    const int oc = (int)(i - p * oc4) * 4;
    const int64_t n = p / OHW;
    const int rem = (int)(p - n * OHW);
    // Every load is issued whatever the channel or slice (clamped, masked afterwards), two slices at a time: a
    // load under a condition waits for the one before it, and this kernel is a few round trips to memory.
    int32_t v[4];
    int64_t at[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int ce = oc + e < g.OC ? oc + e : g.OC - 1;
      at[e] = (n * g.OC + ce) * OHW + rem;
      v[e] = ep.bias ? ep.bias[ce] : 0;
    }
    for (int k0 = 0; k0 < kslices; k0 += 2) {
      const bool two = k0 + 1 < kslices;
      const int32_t* p0 = part + (int64_t)k0 * slice_stride;
      const int32_t* p1 = part + (int64_t)(two ? k0 + 1 : k0) * slice_stride;
      int32_t t0[4], t1[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) { t0[e] = p0[at[e]]; t1[e] = p1[at[e]]; }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = wadd(wadd(v[e], t0[e]), two ? t1[e] : 0);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = oc + e < g.OC ? v[e] : 0;
    run_chain(ep.chain, v);
    if (OUT == OUT_I32_NCHW) {
      int32_t* y32 = reinterpret_cast<int32_t*>(out) + n * ep.o32_img + (int64_t)oc * ep.o32_ch + (int64_t)rem * ep.o32_px;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (oc + e < g.OC) y32[(int64_t)e * ep.o32_ch] = v[e];
    } else {
      uint32_t w[1] = {pack_bytes(v[0], v[1], v[2], v[3])};
      mask_channels(w, oc, g.OC);
      if (oc < ep.out_cp) *reinterpret_cast<uint32_t*>(reinterpret_cast<int8_t*>(out) + act_offset(p, oc, ep.out_cp)) = w[0];
    }
  }
}

constexpr int KSTEP = 64;  // granularity K is padded to

// ---------------------------------------------------------------- packing
// int32 NCHW -> int8 activations (layout of conv_mfma.h, padding channels zero);
// narrowing is static_cast<int8_t>, the reference's own (ops.cc:234).  One
// thread per dword of the destination.
__global__ void __launch_bounds__(256) k_pack_act(const int32_t* __restrict__ x, uint32_t* __restrict__ xp, int64_t total,
                                                  int64_t npix, int c, int hw, int cp) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    int64_t p;
    int c0;
    act_decode(i, cp, &p, &c0);
    if (p >= npix) continue;
    const int64_t n = p / hw;
    const int pix = (int)(p - n * hw);
    // four loads in flight (channels past the last re-read it and are masked afterwards): a load under a
    // condition waits for the one before it
    int32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ch = c0 + j < c ? c0 + j : c - 1;
      v[j] = x[(n * c + ch) * hw + pix];
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t pack = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) pack |= (c0 + j < c ? (uint32_t)(uint8_t)(int8_t)v[j] : 0u) << (8 * j);
    xp[i] = pack;
  }
}

// int32 OIHW -> int8 filter in MFMA-fragment order.  With k = (r*KW + s)*Cp + c the
// matrix [OCp][Kp] is cut into 32-row tiles and 32-byte K chunks; one chunk of
// one tile is stored as the 1 KiB a wavefront feeds to v_mfma_i32_32x32x32_i8:
// lane l holds row (l & 31), bytes (l >> 5)*16 .. +15 of the chunk.  Each tile
// has nch + 1 chunks; the last one is all zero (a K range that ends early reads
// it instead of branching).  Layout: [OCp/32][nch + 1][64][16].
// row_bytes > 0 selects the row-window K order k = kh*row_bytes + kw*4 + c (conv_mfma.h: StemGeom).
__global__ void __launch_bounds__(256) k_pack_weights(const int32_t* __restrict__ w, int8_t* __restrict__ wp, int64_t total,
                                                      int oc, int ic, int taps, int cp, int nch, int row_bytes, int kw_taps) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int d = (int)(i & 3);
    const int lane = (int)((i >> 2) & 63);
    const int64_t t = i >> 8;
    const int chunk = (int)(t % (nch + 1));
    const int64_t tile = t / (nch + 1);
    const int64_t o = tile * 32 + (lane & 31);
    const int k = chunk * 32 + (lane >> 5) * 16 + d * 4;
    int tap = k / cp, c = k - tap * cp;
    if (row_bytes > 0) {
      const int r = k / row_bytes, s4 = (k - r * row_bytes) >> 2;   // filter row, tap inside the window
      tap = s4 < kw_taps ? r * kw_taps + s4 : taps;                  // window bytes past the last tap multiply by zero
      c = 0;
    }
    uint32_t pack = 0;
    if (o < oc && tap < taps && chunk < nch) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int32_t v = (c + j < ic) ? w[((int64_t)o * ic + c + j) * taps + tap] : 0;
        pack |= (uint32_t)(uint8_t)(int8_t)v << (8 * j);
      }
    }
    reinterpret_cast<uint32_t*>(wp)[i] = pack;
  }
}

// int32 NCHW -> row-window input int8 [N][hp][wp][4], zero outside the image (conv_mfma.h: StemGeom)
__global__ void __launch_bounds__(256) k_pack_stem(const int32_t* __restrict__ x, uint32_t* __restrict__ xs, int64_t total,
                                                   int nimg, int c, int h, int w, int hp, int wp, int ph, int pw,
                                                   FastDiv div_wp, FastDiv div_hp) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    // total < 2^31 (checked by the host): 32-bit multiply-high divisions, three instructions each
    const unsigned t = fastdiv((unsigned)i, div_wp);
    const int q = (int)((unsigned)i - t * (unsigned)wp);
    const int64_t n = fastdiv(t, div_hp);
    const int p = (int)(t - (unsigned)n * (unsigned)hp);
    const int ih = p - ph, iw = q - pw;
    // the slack behind the last image and the padding ring are cleared; every thread loads (from the
    // nearest pixel inside, the last channel again past c) so that its loads are all in flight at once
    const bool inside = n < nimg && ih >= 0 && ih < h && iw >= 0 && iw < w;
    const int64_t nc = n < nimg ? n : nimg - 1;
    const int ihc = ih < 0 ? 0 : (ih < h ? ih : h - 1), iwc = iw < 0 ? 0 : (iw < w ? iw : w - 1);
    int32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = x[((nc * c + (j < c ? j : c - 1)) * h + ihc) * w + iwc];
    __builtin_amdgcn_sched_barrier(0);
    uint32_t pack = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) pack |= (j < c ? (uint32_t)(uint8_t)(int8_t)v[j] : 0u) << (8 * j);
    xs[i] = inside ? pack : 0u;
  }
}

// int8 activations -> int32 NCHW
__global__ void __launch_bounds__(256) k_unpack_act(const int8_t* __restrict__ xp, int32_t* __restrict__ x, int64_t total,
                                                    int c, int hw, int cp) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int pix = (int)(i % hw);
    const int64_t t = i / hw;
    const int ch = (int)(t % c);
    const int64_t n = t / c;
    x[i] = xp[act_offset(n * hw + pix, ch, cp)];
  }
}

// ---------------------------------------------------------------- exact int32 paths
// groups > 1 (incl. depthwise): direct convolution on the int32 values, no
// narrowing -- what the reference does for grouped filters (ops.cc:333-366).
__global__ void __launch_bounds__(256)
k_conv_grouped(const int32_t* __restrict__ x, const int32_t* __restrict__ w, const int32_t* __restrict__ bias,
               int32_t* __restrict__ y, int64_t total, int ic, int h, int wd, int oc, int oh, int ow, int kh, int kw,
               int sh, int sw, int ph, int pw, int dh, int dw, int icg, int ocg) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int q = (int)(i % ow);
    const int p = (int)((i / ow) % oh);
    const int o = (int)((i / ((int64_t)ow * oh)) % oc);
    const int64_t b = i / ((int64_t)ow * oh * oc);
    const int cbase = (o / ocg) * icg;
    int32_t acc = 0;
    for (int c = 0; c < icg; ++c) {
      const int32_t* xc = x + ((int64_t)b * ic + cbase + c) * h * wd;
      const int32_t* wc = w + ((int64_t)o * icg + c) * kh * kw;
      for (int r = 0; r < kh; ++r) {
        const int ih = p * sh + r * dh - ph;
        if (ih < 0 || ih >= h) continue;
        for (int t = 0; t < kw; ++t) {
          const int iw = q * sw + t * dw - pw;
          if (iw < 0 || iw >= wd) continue;
          acc = wadd(acc, wmul(xc[(int64_t)ih * wd + iw], wc[r * kw + t]));
        }
      }
    }
    y[i] = wadd(acc, bias ? bias[o] : 0);
  }
}

// dense on int32 operands without narrowing (ops.cc:53-62 multiplies the full int32 values): one
// wavefront per output column j and block of DENSE_MB rows, so a filter row is read once per block.
constexpr int DENSE_MB = 8;
__global__ void __launch_bounds__(256)
k_dense_i32(const int32_t* __restrict__ x, const int32_t* __restrict__ w, const int32_t* __restrict__ bias,
            int32_t* __restrict__ y, int m, int k, int n) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  const int mblocks = (m + DENSE_MB - 1) / DENSE_MB;
  const int64_t total = (int64_t)mblocks * n;
  for (int64_t o = wave; o < total; o += nwaves) {
    const int mb = (int)(o / n);
    const int j = (int)(o - (int64_t)mb * n);
    const int m0 = mb * DENSE_MB;
    const int rows = m - m0 < DENSE_MB ? m - m0 : DENSE_MB;
    const int32_t* wr = w + (int64_t)j * k;
    int32_t acc[DENSE_MB];
#pragma unroll
    for (int r = 0; r < DENSE_MB; ++r) acc[r] = 0;
    // rows past the last one repeat it (their sums are not stored): no load sits under a condition, so the
    // nine loads of a step are in flight together
    const int32_t* xr[DENSE_MB];
#pragma unroll
    for (int r = 0; r < DENSE_MB; ++r) xr[r] = x + (int64_t)(m0 + (r < rows ? r : rows - 1)) * k;
    for (int t = lane; t < k; t += 64) {
      const int32_t wv = wr[t];
      int32_t xv[DENSE_MB];
#pragma unroll
      for (int r = 0; r < DENSE_MB; ++r) xv[r] = xr[r][t];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < DENSE_MB; ++r) acc[r] = wadd(acc[r], wmul(xv[r], wv));
    }
#pragma unroll
    for (int r = 0; r < DENSE_MB; ++r) {
      int32_t a = acc[r];
      for (int d = 32; d >= 1; d >>= 1) a = wadd(a, __shfl_xor(a, d, 64));
      if (lane == 0 && r < rows) y[(int64_t)(m0 + r) * n + j] = wadd(a, bias ? bias[j] : 0);
    }
  }
}

// ---------------------------------------------------------------- host side
// Kernel choice forced by the calling thread (tests and tuning runs); automatic unless set.
static ConvTuning default_tuning() {
  ConvTuning t = {CONV_KERNEL_AUTO, -1, 0, 0, 2000000, nullptr, 0, {}, 1};
  memset(t.seq_layer_cfg, -1, sizeof(t.seq_layer_cfg));
  return t;
}
static thread_local ConvTuning t_conv_tuning = default_tuning();
void set_conv_tuning(const ConvTuning& t) { t_conv_tuning = t; }

int pad_channels(int c) {
  if (c <= 4) return 4;
  if (c <= 8) return 8;
  if (c <= 16) return 16;
  return (c + 31) / 32 * 32;
}

size_t packed_act_bytes(int64_t npix, int c) { return ((size_t)act_bytes(npix, pad_channels(c)) + 255) / 256 * 256; }

// Depthwise filter int32 [C][1][KH][KW] as the MFMA operand of a convolution whose 32 output channels
// of a tile read only their own 32 input channels: per tile, one 1 KiB chunk per tap holding the
// 32x32 diagonal matrix diag(w[c][tap]) in fragment order (lane l: row l & 31, bytes (l >> 5)*16 .. +15
// of K), then the zero chunks up to Kp/32 + 1.  One thread per dword of the destination.
__global__ void __launch_bounds__(256) k_pack_depthwise_diag(const int32_t* __restrict__ w, uint32_t* __restrict__ wp,
                                                             int64_t total, int c, int taps, int nch1) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int dword = (int)(i & 255);            // inside the KiB chunk
    const int64_t chunk_lin = i >> 8;
    const int chunk = (int)(chunk_lin % nch1);
    const int tile = (int)(chunk_lin / nch1);
    const int lane = dword >> 2, part = dword & 3;
    const int row = lane & 31, k0 = (lane >> 5) * 16 + part * 4;   // this dword holds K columns k0 .. k0+3 of the row
    uint32_t v = 0;
    const int ch = tile * 32 + row;
    if (chunk < taps && ch < c && row >= k0 && row < k0 + 4)
      v = (uint32_t)(uint8_t)(int8_t)w[(int64_t)ch * taps + chunk] << (8 * (row - k0));
    wp[i] = v;
  }
}

size_t packed_depthwise_diag_bytes(int c, int kh, int kw) {
  const int kp = (kh * kw * 32 + KSTEP - 1) / KSTEP * KSTEP;
  const int tiles = (c + 127) / 128 * 4;
  return (size_t)tiles * (kp / 32 + 1) * 1024 + 8192;
}

int pack_depthwise_diag(const int32_t* w, int8_t* wp, int c, int kh, int kw, hipStream_t s) {
  const int kp = (kh * kw * 32 + KSTEP - 1) / KSTEP * KSTEP;
  const int64_t total = (int64_t)packed_depthwise_diag_bytes(c, kh, kw) / 4;   // the slack behind the last tile is written as zeros too
  k_pack_depthwise_diag<<<grid_for(total, 256), 256, 0, s>>>(w, reinterpret_cast<uint32_t*>(wp), total, c, kh * kw, kp / 32 + 1);
  return check_launch("pack_depthwise_diag");
}

void weight_dims(int oc, int ic, int kh, int kw, int* ocp, int* kp) {
  const int cp = pad_channels(ic);
  *kp = (kh * kw * cp + KSTEP - 1) / KSTEP * KSTEP;
  *ocp = (oc + 127) / 128 * 128;
}

size_t packed_weight_bytes(int oc, int ic, int kh, int kw) {
  int ocp, kp;
  weight_dims(oc, ic, kh, kw, &ocp, &kp);
  // one zero chunk per 32-row tile, and 8 KiB of slack: the pipelined fetch of
  // the LDS kernel reads up to two K steps past the last tile and never uses them
  return (size_t)(ocp / 32) * (kp / 32 + 1) * 1024 + 8192;
}

size_t packed_weight_pair_bytes(int oc_a, int oc_b, int ic, int kh, int kw) {
  int ocp, kp;
  weight_dims(oc_b, ic, kh, kw, &ocp, &kp);
  // the first filter's tiles, the second one's as pack_weights writes them (rounded up to four), four more that
  // the large-tile kernel's requests may touch, and the slack of packed_weight_bytes
  return (size_t)((oc_a + 31) / 32 + ocp / 32 + 4) * (kp / 32 + 1) * 1024 + 8192;
}

int pack_weights_pair(const int32_t* w_a, int oc_a, const int32_t* w_b, int oc_b, int8_t* wp, int ic, int kh, int kw, hipStream_t s) {
  int ocp, kp;
  weight_dims(oc_a, ic, kh, kw, &ocp, &kp);
  // the first filter is written with its tiles rounded up to four; the second one then overwrites the padding tiles
  const int rc = pack_weights(w_a, wp, oc_a, ic, kh, kw, s);
  if (rc) return rc;
  return pack_weights(w_b, wp + (size_t)((oc_a + 31) / 32) * (kp / 32 + 1) * 1024, oc_b, ic, kh, kw, s);
}

int pack_activations(const int32_t* x, int8_t* xp, int n, int c, int hw, hipStream_t s) {
  const int cp = pad_channels(c);
  const int64_t npix = (int64_t)n * hw;
  const int64_t total = act_bytes(npix, cp) / 4;
  if (total == 0) return CVMHIP_OK;
  KernelTimer timer("k_pack_act", (double)n * c * hw * 5.0, s);  // bytes: 4 read + 1 written per element
  k_pack_act<<<grid_for(total, 256), 256, 0, s>>>(x, reinterpret_cast<uint32_t*>(xp), total, npix, c, hw, cp);
  return check_launch("pack_act");
}

int unpack_activations(const int8_t* xp, int32_t* x, int n, int c, int hw, hipStream_t s) {
  const int64_t total = (int64_t)n * c * hw;
  if (total == 0) return CVMHIP_OK;
  k_unpack_act<<<grid_for(total, 256), 256, 0, s>>>(xp, x, total, c, hw, pad_channels(c));
  return check_launch("unpack_act");
}

int pack_weights(const int32_t* w, int8_t* wp, int oc, int ic, int kh, int kw, hipStream_t s) {
  int ocp, kp;
  weight_dims(oc, ic, kh, kw, &ocp, &kp);
  const int nch = kp / 32;
  const int64_t total = (int64_t)(ocp / 32) * (nch + 1) * 256;  // dwords
  k_pack_weights<<<grid_for(total, 256), 256, 0, s>>>(w, wp, total, oc, ic, kh * kw, pad_channels(ic), nch, 0, kw);
  return check_launch("pack_weights");
}

bool stem_eligible(int c, int kh, int kw, int dil_h, int dil_w) {
  return c >= 1 && c <= 4 && kw * 4 <= 32 && kh >= 1 && dil_h == 1 && dil_w == 1;
}

StemGeom stem_geom(int n, int h, int w, int kh, int kw, int sh, int sw, int ph, int pw) {
  StemGeom sg;
  sg.row_bytes = kw * 4 <= 16 ? 16 : 32;
  sg.k = kh * sg.row_bytes;
  sg.kp = (sg.k + KSTEP - 1) / KSTEP * KSTEP;
  const int oh = (h + 2 * ph - kh) / sh + 1, ow = (w + 2 * pw - kw) / sw + 1;
  // rows and columns the windows of the last output pixel reach (K is rounded up to whole 32-byte chunks)
  const int max_row = (((sg.k + 31) / 32) * 2 - 1) / (sg.row_bytes / 16);
  const int need_h = (oh - 1) * sh + max_row + 1, need_w = (ow - 1) * sw + sg.row_bytes / 4;
  sg.hp = need_h > h + 2 * ph ? need_h : h + 2 * ph;
  sg.wp = need_w > w + 2 * pw ? need_w : w + 2 * pw;
  sg.bytes = ((size_t)n * sg.hp * sg.wp * 4 + 64 + 255) / 256 * 256;   // 64: the last window may run past the last row
  return sg;
}

int pack_stem_input(const int32_t* x, int8_t* xs, int n, int c, int h, int w, int kh, int kw, int sh, int sw, int ph,
                    int pw, hipStream_t s) {
  const StemGeom sg = stem_geom(n, h, w, kh, kw, sh, sw, ph, pw);
  const int64_t total = (int64_t)sg.bytes / 4;   // the slack behind the last row is cleared too
  KernelTimer timer("k_pack_stem", (double)n * c * h * w * 5.0, s);
  if (total > INT32_MAX) return arg_error("pack_stem size");
  k_pack_stem<<<grid_for(total, 256), 256, 0, s>>>(x, reinterpret_cast<uint32_t*>(xs), total, n, c, h, w, sg.hp, sg.wp, ph, pw,
                                                   make_fastdiv((uint32_t)sg.wp), make_fastdiv((uint32_t)sg.hp));
  return check_launch("pack_stem");
}

int pack_stem_weights(const int32_t* w, int8_t* wp, int oc, int c, int kh, int kw, hipStream_t s) {
  const int rb = kw * 4 <= 16 ? 16 : 32;
  const int kp = (kh * rb + KSTEP - 1) / KSTEP * KSTEP;
  const int ocp = (oc + 127) / 128 * 128;
  const int nch = kp / 32;
  const int64_t total = (int64_t)(ocp / 32) * (nch + 1) * 256;  // dwords
  k_pack_weights<<<grid_for(total, 256), 256, 0, s>>>(w, wp, total, oc, c, kh * kw, 4, nch, rb, kw);
  return check_launch("pack_stem_weights");
}

size_t packed_stem_weight_bytes(int oc, int kp) { return (size_t)((oc + 127) / 128 * 128 / 32) * (kp / 32 + 1) * 1024 + 8192; }


template <int WM, int WN, int OUT>
static void launch_tile(int gran, bool wide, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out,
                        const ConvGeom& g, const Epilogue& ep) {
  if (gran == 16) {
    // 128-byte K steps halve the number of barriers; the 128x128 tile keeps 64 (LDS budget)
    if constexpr (WM + WN < 4) {
      if (wide) {
        k_conv_igemm<WM, WN, 16, 128, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
        return;
      }
    }
    k_conv_igemm<WM, WN, 16, 64, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
  } else if (gran == 8) {
    k_conv_igemm<WM, WN, 8, 64, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
  } else {
    k_conv_igemm<WM, WN, 4, 64, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
  }
}

template <int OUT>
static void launch_out(int wm, int wn, int gran, bool wide, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp,
                       void* out, const ConvGeom& g, const Epilogue& ep) {
  if (wm == 2 && wn == 2) launch_tile<2, 2, OUT>(gran, wide, grid, s, xp, wp, out, g, ep);
  else if (wm == 1 && wn == 2) launch_tile<1, 2, OUT>(gran, wide, grid, s, xp, wp, out, g, ep);
  else if (wm == 2 && wn == 1) launch_tile<2, 1, OUT>(gran, wide, grid, s, xp, wp, out, g, ep);
  else launch_tile<1, 1, OUT>(gran, wide, grid, s, xp, wp, out, g, ep);
}

// ---- wavefront-private kernel: configurations and choice
struct WaveCfg { int tm, tn, ksplit, nw, blocks_per_cu; };
static const WaveCfg kWaveCfgs[] = {
    // tile rows x cols of 32, K split, wavefronts, resident workgroups per CU (registers and LDS)
    {2, 2, 8, 8, 1}, {2, 2, 4, 4, 2}, {2, 2, 2, 4, 2}, {2, 2, 1, 4, 2},
    {1, 2, 8, 8, 2}, {1, 2, 4, 4, 2}, {1, 2, 1, 4, 2},
    {2, 4, 1, 4, 2},
};
constexpr int kNumWaveCfgs = sizeof(kWaveCfgs) / sizeof(kWaveCfgs[0]);

template <int TM, int TN, int KSPLIT, int NW, int D, int MINW, int OUT>
static void launch_wave_mode(int mode, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out,
                             const ConvGeom& g, const Epilogue& ep) {
  if (mode == WAVE_IDENT) k_conv_wave<TM, TN, KSPLIT, NW, D, MINW, OUT, WAVE_IDENT><<<grid, NW * 64, 0, s>>>(xp, wp, out, g, ep);
  else if (mode == WAVE_NOPAD) k_conv_wave<TM, TN, KSPLIT, NW, D, MINW, OUT, WAVE_NOPAD><<<grid, NW * 64, 0, s>>>(xp, wp, out, g, ep);
  else if (mode == WAVE_ROWS) k_conv_wave<TM, TN, KSPLIT, NW, D, MINW, OUT, WAVE_ROWS><<<grid, NW * 64, 0, s>>>(xp, wp, out, g, ep);
  else k_conv_wave<TM, TN, KSPLIT, NW, D, MINW, OUT, WAVE_PAD><<<grid, NW * 64, 0, s>>>(xp, wp, out, g, ep);
}

// K-sliced launch: 32-channel tiles, 8-way K split inside the workgroup, raw int32 partial sums (no row-window mode)
static void launch_wave_sliced(int mode, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out,
                               const ConvGeom& g, const Epilogue& ep) {
  // At most 32 pixels (a dense layer at a batch of up to 32): one pixel block per tile instead of two, of which the second
  // would be all padding and still cost its requests, and K split over four wavefronts instead of eight, so that a
  // wavefront streams twice as long a run of the filter (VGG-16's first dense layer at batch 16, 103 MB of filter:
  // 27.2 -> 21.8-22.9 us, 3.8 -> 4.6 TB/s; with eight K slices over the grid instead of four 23.4 us).
  if (mode == WAVE_IDENT && g.P <= 32) {
    k_conv_wave<1, 1, 4, 4, 4, 2, OUT_I32_NCHW, WAVE_IDENT, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
    return;
  }
  if (mode == WAVE_IDENT) k_conv_wave<1, 2, 8, 8, 4, 2, OUT_I32_NCHW, WAVE_IDENT, true><<<grid, 512, 0, s>>>(xp, wp, out, g, ep);
  else if (mode == WAVE_NOPAD) k_conv_wave<1, 2, 8, 8, 4, 2, OUT_I32_NCHW, WAVE_NOPAD, true><<<grid, 512, 0, s>>>(xp, wp, out, g, ep);
  else k_conv_wave<1, 2, 8, 8, 4, 2, OUT_I32_NCHW, WAVE_PAD, true><<<grid, 512, 0, s>>>(xp, wp, out, g, ep);
}

template <int TM, int TN, int KSPLIT, int NW, int D, int MINW>
static void launch_wave_cfg(int mode, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out,
                            const ConvGeom& g, const Epilogue& ep) {
  if (ep.out_mode == OUT_I8_ACT) launch_wave_mode<TM, TN, KSPLIT, NW, D, MINW, OUT_I8_ACT>(mode, grid, s, xp, wp, out, g, ep);
  else launch_wave_mode<TM, TN, KSPLIT, NW, D, MINW, OUT_I32_NCHW>(mode, grid, s, xp, wp, out, g, ep);
}

static int64_t wave_cfg_blocks(const WaveCfg& c, const ConvGeom& g) {
  const int bm = 32 * c.tm, bn = 32 * c.tn * (c.nw / c.ksplit);
  return (int64_t)((g.OC + bm - 1) / bm) * ((g.P + bn - 1) / bn);
}

// A wavefront that runs alone pays full latency for every instruction and every
// load, so the aim is one round of workgroups with as little serial K per
// wavefront as possible: the deepest K split (at least two chunks per wavefront)
// of the largest tile whose grid is resident at once.  Larger grids run unsplit
// in several rounds (the wavefronts of a workgroup then share the filter through L1).
// `cus`: compute units the layer runs on (the chip, or one XCD for a share of a layer-sequence launch; g.P is then the share's)
static int choose_wave_cfg_base(const ConvGeom& g, int cus);
// The choice below, corrected for layers it leaves on fewer than half of the chip (few pixels and a short K, for
// which the rule "at least two chunks per wavefront" rules out every K split: 64 -> 256 channels at 56 x 56 at
// batch 1 is 52 workgroups of 64 x 256): a configuration whose grid lands between half of the CUs and all of them
// is taken instead, the one with the shallowest split among those -- some of its wavefronts then have no K chunk of
// their own, which costs less than idle CUs (batch-1 ResNet-50: 263 -> 247 us per step).
static int choose_wave_cfg(const ConvGeom& g, int cus = 256) {
  const int base = choose_wave_cfg_base(g, cus);
  if (cus != 256 || g.OC <= 32 || base == 7 || wave_cfg_blocks(kWaveCfgs[base], g) >= cus / 2) return base;
  static const int order[] = {3, 2, 1, 6, 5, 0, 4};   // by K split, 64-channel tiles first
  for (int i : order) {
    const int64_t b = wave_cfg_blocks(kWaveCfgs[i], g);
    if (b >= cus / 2 && b <= cus) return i;
  }
  return base;
}
static int choose_wave_cfg_base(const ConvGeom& g, int cus) {
  const int nlive = g.K / 32;
  // very few pixels, deep K (fully connected layers, the last stage): even the deepest split of
  // the 64-channel tile leaves SIMDs without a wavefront, so halve the tile instead
  // (one XCD's share of a layer-sequence launch: also when the 64-channel tiles would fill exactly half of its 32 CUs --
  // the 512-channel layers of a ResNet's last stage, 16 tiles -- where the 32 tiles of the halved tile give every CU
  // 0.75 of the operand bytes instead of every second CU all of them: 363 -> 355 us for the ResNet-50 sequence)
  if (g.OC > 32 && nlive >= 16 && wave_cfg_blocks(kWaveCfgs[0], g) < cus / 2 + (cus == 32 ? 1 : 0)) return 4;
  const int first = g.OC > 32 ? 0 : 4;
  const int last = g.OC > 32 ? 4 : 7;   // 64-channel tiles: 0..3 (and 7, see below); 32-channel tiles: 4..6
  for (int i = first; i < last; ++i) {
    const WaveCfg& c = kWaveCfgs[i];
    if (c.ksplit > 1 && nlive < 2 * c.ksplit) continue;
    const int64_t capacity = cus * (int64_t)c.blocks_per_cu;
    if (c.ksplit == 1 || wave_cfg_blocks(c, g) <= capacity) {
      // Unsplit with a grid of many rounds and a long K loop (the large layers of a VGG): the K loop is bound by
      // operand delivery, and a 64 x 128 wavefront tile takes 0.75 KiB per MFMA instead of 1 KiB (measured
      // 1.0 -> 1.2-1.3 POP/s on 28x28x512 and 56x56x256 layers with 3x3 filters).
      if (cus == 256 && c.ksplit == 1 && g.OC > 32 && g.K >= 512 && wave_cfg_blocks(kWaveCfgs[7], g) >= 192) return 7;
      // Unsplit, short K, between one and two rounds of 64 x 64 tiles (ResNet's input layer: 784 workgroups for 512
      // places): the second round is half empty, while the 64 x 128 tile fits one round (10.0 against 11.9 us)
      if (cus == 256 && c.ksplit == 1 && g.OC > 32 && i == 3) {
        const int64_t small = wave_cfg_blocks(c, g), big = wave_cfg_blocks(kWaveCfgs[7], g);
        const int64_t places = capacity;
        if (small > places && small <= 2 * places && big <= places) return 7;
      }
      return i;
    }
  }
  return last - 1;
}

// ---- large-tile kernel: tile shapes and choice
struct BigCfg { int wgm, wgn, tm, tn; };
static const BigCfg kBigCfgs[] = {{2, 2, 4, 4}, {2, 2, 2, 4}, {1, 4, 2, 4}};   // 256x256, 128x256, 64x512 (channels x pixels)
static int64_t big_cfg_blocks(const BigCfg& c, const ConvGeom& g) {
  const int bm = c.wgm * c.tm * 32, bn = c.wgn * c.tn * 32;
  return (int64_t)((g.OC + bm - 1) / bm) * ((g.P + bn - 1) / bn);
}
// The largest tile that does not reach past the layer's channels and still gives most compute units a tile; -1 when
// the layer is too small for this kernel (fewer than 160 tiles of the smallest fitting shape, or a short K).
static int choose_big_cfg(const ConvGeom& g) {
  // K >= 512: with K = 256 (the 1x1 layers of a ResNet's second stage) the ring never fills and the wavefront
  // kernel is faster (7.5 us against 11.6 for 256 -> 128 channels over 16 x 56 x 56 pixels)
  if (g.dw || g.row_bytes || (g.Cp % 32) != 0 || g.KH > 32 || g.KW > 32 || g.K < 512) return -1;
  // 128 x 256 tiles, two workgroups per compute unit, measured best (1.4-1.6 POP/s on the 3x3 layers of a VGG against
  // 1.05-1.2 for the wavefront kernel); the 256 x 256 tile (one workgroup, 1.4) and the 64 x 512 one (0.65, below the
  // wavefront kernel's 0.96 on 64 -> 64 channels) are kept for forced use
  if (g.OC <= 64) return -1;
  return big_cfg_blocks(kBigCfgs[1], g) >= 160 ? 1 : -1;
}
template <int OUT>
static void launch_big_out(int cfg, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out, const ConvGeom& g,
                           const Epilogue& ep) {
  if constexpr (OUT == OUT_I8_ACT) {
    if (ep.pool == 2) {   // the maximum of a fused 2x2 pool between registers: instantiations of their own
      if (cfg == 0) k_conv_big<2, 2, 4, 4, OUT, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
      else if (cfg == 1) k_conv_big<2, 2, 2, 4, OUT, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
      else k_conv_big<1, 4, 2, 4, OUT, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
      return;
    }
  }
  if (cfg == 0) k_conv_big<2, 2, 4, 4, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
  else if (cfg == 1) k_conv_big<2, 2, 2, 4, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
  else k_conv_big<1, 4, 2, 4, OUT><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
}

static void launch_wave(int cfg, int mode, unsigned grid, hipStream_t s, const int8_t* xp, const int8_t* wp, void* out,
                        const ConvGeom& g, const Epilogue& ep) {
  switch (cfg) {
    case 0: launch_wave_cfg<2, 2, 8, 8, 2, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 1: launch_wave_cfg<2, 2, 4, 4, 2, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 2: launch_wave_cfg<2, 2, 2, 4, 2, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 3: launch_wave_cfg<2, 2, 1, 4, 2, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 4: launch_wave_cfg<1, 2, 8, 8, 4, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 5: launch_wave_cfg<1, 2, 4, 4, 4, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    case 6: launch_wave_cfg<1, 2, 1, 4, 4, 2>(mode, grid, s, xp, wp, out, g, ep); break;
    default:
      if (ep.pool == 2 && ep.out_mode == OUT_I8_ACT) {   // the maximum of a fused 2x2 pool between registers (never the row-window or 1x1-identity mode)
        if (mode == WAVE_NOPAD) k_conv_wave<2, 4, 1, 4, 1, 2, OUT_I8_ACT, WAVE_NOPAD, false, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
        else k_conv_wave<2, 4, 1, 4, 1, 2, OUT_I8_ACT, WAVE_PAD, false, true><<<grid, 256, 0, s>>>(xp, wp, out, g, ep);
        break;
      }
      launch_wave_cfg<2, 4, 1, 4, 1, 2>(mode, grid, s, xp, wp, out, g, ep);
      break;
  }
}

// K slices over the grid: for a layer with at most 64 output pixels and K >= 8192 (a fully connected layer at a
// small batch) the filter stream is the whole cost, and one workgroup per 32 output channels is too few
// workgroups to keep it flowing.  Returns the number of slices (1 = not applicable).
static int conv_slices(const ConvGeom& g, const Epilogue& ep) {
  const int64_t p = (int64_t)g.N * g.OH * g.OW;
  const int64_t k = (int64_t)g.KH * g.KW * g.Cp;
  if (g.dw || g.row_bytes || (g.Cp % 32) != 0 || p > 64 || k < 8192 || g.OC < 32 || ep.residual) return 1;
  if (!(g.PH == 0 && g.PW == 0) && (g.KH > 32 || g.KW > 32)) return 1;
  const int tiles = (g.OC + 31) / 32;
  if (tiles > 256) return 1;
  return tiles <= 128 ? 4 : 2;   // a power of two: the slice is the low bits of the block index
}

size_t conv_slices_workspace_bytes(const ConvGeom& g, const Epilogue& ep) {
  const int ks = conv_slices(g, ep);
  return ks > 1 ? (size_t)ks * g.N * g.OC * g.OH * g.OW * 4 : 0;
}

// Algorithmic HBM bytes of a convolution launch (true channels, each tensor once) and a one-line description
// of it, for the measurement harness (only evaluated while kernel timing is on).
static double conv_bytes(const ConvGeom& g, const Epilogue& ep) {
  const double c = g.C ? g.C : g.Cp;
  const double in = (double)g.N * g.H * g.W * (g.row_bytes ? 4.0 : c);
  const double flt = (double)g.OC * (g.dw ? 1.0 : c) * g.taps;
  const double outb = (double)g.P * g.OC * (ep.out_mode == OUT_I8_ACT ? 1.0 : 4.0) / (ep.pool ? 4.0 : 1.0);
  return in + flt + outb + (ep.residual ? (double)g.P * g.OC : 0.0);
}
struct ConvDesc {
  char text[160];
  ConvDesc(const ConvGeom& g, const Epilogue& ep, const char* kernel, int cfg, int mode, long grid) {
    text[0] = 0;
    if (!kernel_timing_enabled()) return;
    snprintf(text, sizeof(text), "%s%dx%d/%d %d->%d in %dx%dx%d out %dx%d%s%s %s cfg %d mode %d grid %ld", g.dw ? "dw " : "",
             g.KH, g.KW, g.SH, g.C ? g.C : g.Cp, g.OC, g.N, g.H, g.W, g.OH, g.OW, ep.residual ? " +res" : ep.pool ? " +pool" : "",
             ep.out_mode == OUT_I8_ACT ? " i8" : " i32", kernel, cfg, mode, grid);
  }
};

int conv_igemm(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep_in, hipStream_t s) {
  return conv_igemm_ws(xp, wp, out, g, ep_in, nullptr, 0, s);
}

bool conv_pool_eligible(const ConvGeom& g) {
  return !g.dw && g.row_bytes == 0 && (g.Cp % 32) == 0 && (pad_channels(g.OC) % 32) == 0 && g.KH <= 32 && g.KW <= 32 &&
         g.OH >= 2 && g.OW >= 2 && (g.OH % 2) == 0 && (g.OW % 2) == 0;
}

// Checks a convolution's geometry and fills the derived fields of g and the defaults of the epilogue.
static int conv_prepare(const int8_t* xp, const int8_t* wp, void* out, ConvGeom& g, const Epilogue& ep_in, Epilogue& ep) {
  const Epilogue& ep0 = ep_in;
  if (g.N < 1 || g.H < 1 || g.W < 1 || g.OC < 1 || g.OH < 1 || g.OW < 1 || g.KH < 1 || g.KW < 1 || g.SH < 1 ||
      g.SW < 1 || g.DH < 1 || g.DW < 1 || g.PH < 0 || g.PW < 0)
    return arg_error("conv geometry");
  if (g.Cp != 4 && g.Cp != 8 && g.Cp != 16 && (g.Cp % 32) != 0) return arg_error("conv channel padding");
  if (g.row_bytes != 0 && (g.Cp != 4 || (g.row_bytes != 16 && g.row_bytes != 32) || g.PH != 0 || g.PW != 0 || g.KW * 4 > g.row_bytes))
    return arg_error("conv row-window geometry");
  if (((uintptr_t)xp | (uintptr_t)wp) & 15) return arg_error("conv operand alignment");
  if ((ep0.out_mode == OUT_I8_ACT || ep0.residual) && ep0.out_cp != pad_channels(g.OC))
    return arg_error("conv int8 output layout");
  if (((uintptr_t)out | (uintptr_t)ep0.residual) & 3) return arg_error("conv output alignment");
  if (ep0.out_mode == OUT_I8_ACT && ep0.out_cp >= 16 && ((uintptr_t)out & 15)) return arg_error("conv output alignment");
  if (g.dw && ((g.Cp % 32) != 0 || g.row_bytes != 0 || g.OC > g.Cp || g.KH > 32 || g.KW > 32))
    return arg_error("depthwise geometry (channels padded to 32, filter side at most 32)");
  g.taps = g.KH * g.KW;
  g.K = g.row_bytes ? g.KH * g.row_bytes : g.dw ? g.taps * 32 : g.taps * g.Cp;
  g.Kp = (g.K + KSTEP - 1) / KSTEP * KSTEP;
  g.P = (int64_t)g.N * g.OH * g.OW;
  // operands are addressed with 32-bit offsets from the tensor's base
  if (act_bytes((int64_t)g.N * g.H * g.W, g.Cp) > INT32_MAX || g.P > INT32_MAX ||
      (int64_t)((g.OC + 127) / 128 * 4) * (g.Kp / 32 + 1) * 1024 > INT32_MAX)
    return arg_error("conv tensor too large");
  ep = ep_in;
  ep.bias_vec = ep.bias != nullptr && ((uintptr_t)ep.bias & 15) == 0;
  ep.chain_flags = chain_flags_of(ep.chain);
  ep.chain2_flags = chain_flags_of(ep.chain2);
  if (ep.o32_img == 0 && ep.o32_ch == 0 && ep.o32_px == 0) {  // int32 output defaults to NCHW
    ep.o32_img = (int64_t)g.OC * g.OH * g.OW;
    ep.o32_ch = g.OH * g.OW;
    ep.o32_px = 1;
  } else if (ep.o32_ch < 1 || ep.o32_px < 1 || ep.o32_img < 0) {
    return arg_error("conv int32 output strides");
  }
  if (ep.split) {
    if (ep.out_mode != OUT_I32_NCHW || ep.residual || ep.pool || ep.split < 32 || (ep.split % 32) != 0 || ep.oc_a < 1 ||
        ep.oc_a > ep.split || ep.oc_b < 1 || g.OC != ep.split + ep.oc_b || !ep.out_b || ((uintptr_t)ep.out_b & 3) ||
        ep.o32_ch_b < 1 || ep.o32_px_b < 1 || ep.o32_img_b < 0 || g.dw || g.row_bytes)
      return arg_error("conv with two int32 destinations: bad split");
  }
  if (ep.pool) {   // pixels are numbered window by window (conv_out_pixel)
    if (!conv_pool_eligible(g) || ep.out_mode != OUT_I8_ACT || ep.residual)
      return arg_error("conv with fused 2x2 max-pool: not eligible (int8 pixel-blocked tensors, even output extent, no residual)");
    g.div_ohw = make_fastdiv((uint32_t)(g.OH * g.OW / 4));
    g.div_ow = make_fastdiv((uint32_t)(g.OW / 2));
  } else {
    g.div_ohw = make_fastdiv((uint32_t)(g.OH * g.OW));
    g.div_ow = make_fastdiv((uint32_t)g.OW);
  }
  g.div_ct = make_fastdiv((uint32_t)(g.dw ? 1 : g.Cp >= 32 ? g.Cp / 32 : 1));
  g.div_kw = make_fastdiv((uint32_t)g.KW);
  return CVMHIP_OK;
}

int conv_igemm_ws(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep_in, void* ws, size_t ws_bytes,
                  hipStream_t s) {
  Epilogue ep;
  const int prc = conv_prepare(xp, wp, out, g, ep_in, ep);
  if (prc) return prc;
  const bool wide = (g.Kp % 128) == 0;
  const int gran = g.Cp >= 16 ? 16 : g.Cp;
  // Tile choice: the largest tile that still yields >= 2 workgroups per CU;
  // small layers fall back to smaller tiles to keep all 256 CUs busy.
  auto blocks = [&](int bm, int bn) { return (int64_t)((g.OC + bm - 1) / bm) * ((g.P + bn - 1) / bn); };
  int wm = g.OC > 64 ? 2 : 1, wn = 2;
  if (blocks(64 * wm, 64 * wn) < 512 && wn == 2) wn = 1;
  if (blocks(64 * wm, 64 * wn) < 512 && wm == 2) wm = 1;
  // test and tuning hook (cvmhip_set_conv_tuning): a forced tile shape of the tiled kernel
  const ConvTuning tune = t_conv_tuning;
  if (tune.tile_wm >= 1 && tune.tile_wm <= 2 && tune.tile_wn >= 1 && tune.tile_wn <= 2) {
    wm = tune.tile_wm;
    wn = tune.tile_wn;
  }
  // kernel choice: the wavefront-private kernel when the layout allows it and its grid fits the chip,
  // else the LDS-tiled kernel.  The calling thread's tuning (cvmhip_set_conv_tuning) can force one of
  // them or a configuration of the wavefront kernel; nothing is read from the environment here.
  const bool force_lds = tune.kernel == CONV_KERNEL_LDS, force_wave = tune.kernel == CONV_KERNEL_WAVE;
  const int wave_forced = tune.wave_cfg;
  const bool nopad = g.PH == 0 && g.PW == 0;
  const bool rows = g.row_bytes != 0;
  const bool wave_ok = rows || ((g.Cp % 32) == 0 && (nopad || (g.KH <= 32 && g.KW <= 32)));
  int cfg = wave_ok ? choose_wave_cfg(g) : -1;
  if (g.dw) {
    // one 32-channel tile per workgroup (its K is its own channels): the 32-row configurations, unsplit
    // unless the grid leaves most of the chip idle
    if (!wave_ok) return arg_error("depthwise geometry");
    cfg = wave_cfg_blocks(kWaveCfgs[6], g) >= 192 || g.taps < 8 ? 6 : 5;
    if (wave_forced >= 4 && wave_forced <= 6) cfg = wave_forced;
  } else
  if (force_lds && !rows) cfg = -1;
  if (wave_ok && force_wave && cfg < 0) cfg = g.OC > 32 ? 3 : 6;
  if (wave_ok && cfg >= 0 && wave_forced >= 0 && wave_forced < kNumWaveCfgs) cfg = wave_forced;
  if (ep.pool && cfg < 0) cfg = g.OC > 32 ? 3 : 6;   // the tiled kernel has no pooled form
  // The pool's maximum can be taken between registers (Epilogue::pool = 2, set below for kernels whose wavefront tile
  // is four pixel blocks wide) when whole wavefront tiles cover the pixels and the chain never decreases as its input
  // grows, which holds for every stage without a multiplication.
  bool pool_in_registers = ep.pool != 0 && (g.P % 128) == 0;
  for (int t = 0; t < ep.chain.count; ++t) pool_in_registers = pool_in_registers && ep.chain.st[t].mul == 1;
  const int kslices = ws && !ep.pool && !ep.split ? conv_slices(g, ep) : 1;
  if (kslices > 1 && wave_ok) {
    const size_t need = (size_t)kslices * g.N * g.OC * g.OH * g.OW * 4;
    if (ws_bytes < need || ((uintptr_t)ws & 15)) return arg_error("conv K-slice workspace");
    cfg = 4;
    const int mode = (g.KH == 1 && g.KW == 1 && g.SH == 1 && g.SW == 1 && nopad && g.OH == g.H && g.OW == g.W)
                         ? WAVE_IDENT : nopad ? WAVE_NOPAD : WAVE_PAD;
    const int64_t wnb = wave_cfg_blocks(kWaveCfgs[cfg], g);
    g.octiles = (g.OC + 31) / 32;
    g.div_octiles = make_fastdiv((uint32_t)g.octiles);
    g.kslices = kslices;
    g.slice_shift = kslices == 4 ? 2 : 1;
    g.slice_chunks = ((g.K + 31) / 32 + kslices - 1) / kslices;
    g.slice_stride = (int)((int64_t)g.N * g.OC * g.OH * g.OW);   // at most 64 pixels x OC
    Epilogue raw = {};                 // slices store raw int32 sums, NCHW, into their plane of the workspace
    raw.out_mode = OUT_I32_NCHW;
    raw.out_cp = ep.out_cp;
    raw.o32_img = (int64_t)g.OC * g.OH * g.OW;
    raw.o32_ch = g.OH * g.OW;
    raw.o32_px = 1;
    {
      const ConvDesc desc(g, ep, "wave-sliced", cfg, mode, (long)(wnb * kslices));
      KernelTimer timer("k_conv_wave", 2.0 * (double)g.P * g.OC * (double)g.taps * (double)(g.C ? g.C : g.Cp), s, conv_bytes(g, ep), desc.text);
      launch_wave_sliced(mode, (unsigned)(wnb * kslices), s, xp, wp, ws, g, raw);
    }
    int rc = check_launch("conv_wave (K slices)");
    if (rc) return rc;
    const int64_t total = g.P * (ep.out_mode == OUT_I8_ACT ? ep.out_cp / 4 : (g.OC + 3) / 4);
    if (ep.out_mode == OUT_I8_ACT)
      k_slices_finish<OUT_I8_ACT><<<grid_for(total, 256), 256, 0, s>>>(reinterpret_cast<const int32_t*>(ws), out, kslices, g.slice_stride, g, ep);
    else
      k_slices_finish<OUT_I32_NCHW><<<grid_for(total, 256), 256, 0, s>>>(reinterpret_cast<const int32_t*>(ws), out, kslices, g.slice_stride, g, ep);
    return check_launch("conv K-slice finish");
  }
  // layers that fill the chip several times over: the large-tile kernel (CONV_KERNEL_BIG forces it where it applies,
  // a forced wavefront or tiled kernel keeps it away)
  {
    const int big = (tune.kernel == CONV_KERNEL_AUTO || tune.kernel == CONV_KERNEL_BIG) && wave_forced < 0 ? choose_big_cfg(g) : -1;
    int bcfg = big;
    if (tune.kernel == CONV_KERNEL_BIG && bcfg < 0 && !g.dw && !rows && (g.Cp % 32) == 0 && g.KH <= 32 && g.KW <= 32)
      bcfg = g.OC > 128 ? 0 : g.OC > 64 ? 1 : 2;   // forced: any size
    if (tune.kernel == CONV_KERNEL_BIG && tune.tile_wm >= 1 && tune.tile_wm <= 3 && bcfg >= 0) bcfg = tune.tile_wm - 1;
    if (bcfg >= 0 && kslices <= 1) {
      const BigCfg& c = kBigCfgs[bcfg];
      if (pool_in_registers && c.tn == 4) ep.pool = 2;
      const int64_t nbig = big_cfg_blocks(c, g);
      if (nbig > 0x7fffffff) return arg_error("conv grid too large");
      g.octiles = (g.OC + c.wgm * c.tm * 32 - 1) / (c.wgm * c.tm * 32);
      g.div_octiles = make_fastdiv((uint32_t)g.octiles);
      const ConvDesc desc(g, ep, "big", bcfg, 0, (long)nbig);
      KernelTimer timer("k_conv_big", 2.0 * (double)g.P * g.OC * (double)g.taps * (double)(g.C ? g.C : g.Cp), s, conv_bytes(g, ep),
                        desc.text);
      if (ep.out_mode == OUT_I8_ACT) launch_big_out<OUT_I8_ACT>(bcfg, (unsigned)nbig, s, xp, wp, out, g, ep);
      else launch_big_out<OUT_I32_NCHW>(bcfg, (unsigned)nbig, s, xp, wp, out, g, ep);
      return check_launch("conv_big");
    }
  }
  if (cfg >= 0) {
    // (with a fused max-pool the pixels are renumbered, so output block t is no longer input block t)
    const int mode = rows ? WAVE_ROWS
                          : (!g.dw && !ep.pool && g.KH == 1 && g.KW == 1 && g.SH == 1 && g.SW == 1 && nopad && g.OH == g.H && g.OW == g.W)
                                ? WAVE_IDENT : nopad ? WAVE_NOPAD : WAVE_PAD;
    const int64_t wnb = wave_cfg_blocks(kWaveCfgs[cfg], g);
    if (wnb > 0x7fffffff) return arg_error("conv grid too large");
    if (pool_in_registers && kWaveCfgs[cfg].tn == 4 && kWaveCfgs[cfg].ksplit == 1) ep.pool = 2;
    g.octiles = (g.OC + 32 * kWaveCfgs[cfg].tm - 1) / (32 * kWaveCfgs[cfg].tm);
    g.div_octiles = make_fastdiv((uint32_t)g.octiles);
    const ConvDesc desc(g, ep, "wave", cfg, mode, (long)wnb);
    KernelTimer timer("k_conv_wave", 2.0 * (double)g.P * g.OC * (double)g.taps * (g.dw ? 1.0 : (double)(g.C ? g.C : g.Cp)), s,
                      conv_bytes(g, ep), desc.text);
    launch_wave(cfg, mode, (unsigned)wnb, s, xp, wp, out, g, ep);
    return check_launch("conv_wave");
  }
  const int64_t nb = blocks(64 * wm, 64 * wn);
  if (nb > 0x7fffffff) return arg_error("conv grid too large");
  const unsigned grid = (unsigned)nb;
  // algorithmic work of this launch: 2 * pixels * OC * (true channels * taps); padding not counted
  const ConvDesc desc(g, ep, "lds", wm * 10 + wn, gran, (long)nb);
  KernelTimer timer("k_conv_igemm", 2.0 * (double)g.P * g.OC * (double)g.taps * (double)(g.C ? g.C : g.Cp), s, conv_bytes(g, ep),
                    desc.text);
  const int ks = (wide && wm + wn < 4) ? 128 : 64;
  g.adv_c = ks % g.Cp;
  g.adv_tap = ks / g.Cp;
  g.adv_r = g.adv_tap / g.KW;
  g.adv_s = g.adv_tap % g.KW;
  if (ep.out_mode == OUT_I8_ACT) launch_out<OUT_I8_ACT>(wm, wn, gran, wide, grid, s, xp, wp, out, g, ep);
  else launch_out<OUT_I32_NCHW>(wm, wn, gran, wide, grid, s, xp, wp, out, g, ep);
  return check_launch("conv_igemm");
}


// ---- row-window convolution + 3x3 stride-2 max-pool: host side
// Pool geometry is fixed (3x3, stride 2, padding 1); qh, qw are the pool's output extent as the graph gives it.
bool stem_pool_eligible(int c, int oc, int kh, int kw, int oh, int ow, int qh, int qw) {
  return stem_eligible(c, kh, kw, 1, 1) && oc >= 32 && oc <= 64 && (oc % 32) == 0 && oh >= 1 && ow >= 1 && qh >= 1 && qw >= 1 &&
         2 * (qh - 1) - 1 <= oh - 1 && 2 * (qw - 1) - 1 <= ow - 1;   // every window touches the convolution's output
}
int stem_pool(const int8_t* xs, const int8_t* wp, const int32_t* bias, const DevChain& chain, int8_t* out, int n, int c, int h,
              int w, int oc, int kh, int kw, int sh, int sw, int ph, int pw, int qh, int qw, hipStream_t s) {
  const int oh = (h + 2 * ph - kh) / sh + 1, ow = (w + 2 * pw - kw) / sw + 1;
  if (!stem_pool_eligible(c, oc, kh, kw, oh, ow, qh, qw)) return arg_error("conv2d_stem_pool3_i8: not eligible");
  if (((uintptr_t)xs | (uintptr_t)wp | (uintptr_t)out) & 15) return arg_error("conv2d_stem_pool3_i8 alignment");
  const StemGeom sg = stem_geom(n, h, w, kh, kw, sh, sw, ph, pw);
  StemPool a = {};
  a.N = n; a.Hs = sg.hp; a.Ws = sg.wp;
  a.OH = oh; a.OW = ow; a.QH = qh; a.QW = qw;
  a.SH = sh; a.SW = sw; a.OC = oc; a.ocp = pad_channels(oc);
  a.nch = sg.kp / 32;
  a.nlive = (sg.k + 31) / 32;
  a.sh16 = sg.row_bytes >> 5;
  a.tiles_x = (qw + SP_PW - 1) / SP_PW;
  a.tiles_y = (qh + SP_PH - 1) / SP_PH;
  a.chain = chain;
  a.bias = bias;
  if (n > 65535 || a.tiles_y > 65535 || sg.bytes > INT32_MAX) return arg_error("conv2d_stem_pool3_i8: tensor too large");
  char desc[128] = "";
  if (kernel_timing_enabled())
    snprintf(desc, sizeof(desc), "%dx%d/%d %d->%d in %dx%dx%d out %dx%d + 3x3/2 max-pool -> %dx%d", kh, kw, sh, c, oc, n, h, w, oh, ow, qh, qw);
  KernelTimer timer("k_stem_pool", 2.0 * n * (double)oh * ow * oc * c * kh * kw, s,
                    4.0 * n * sg.hp * sg.wp + (double)oc * c * kh * kw + (double)n * qh * qw * oc, desc);
  k_stem_pool<<<dim3((unsigned)a.tiles_x, (unsigned)a.tiles_y, (unsigned)n), 256, 0, s>>>(xs, wp, out, a);
  return check_launch("conv2d_stem_pool3_i8");
}

// ---- independent convolutions in one launch: host side
// Fills entry `index` of a host copy of the table for a convolution with int32 output; its workgroups are
// first_block .. first_block + *blocks - 1 of the launch.  CVMHIP_ERR_ARG "not eligible" when the layer cannot be one.
int conv_group_layer(void* table, int index, int first_block, const int8_t* xp, const int8_t* wp, void* out, ConvGeom g,
                     const Epilogue& ep_in, int* blocks) {
  Epilogue ep;
  const int prc = conv_prepare(xp, wp, out, g, ep_in, ep);
  if (prc) return prc;
  const bool nopad = g.PH == 0 && g.PW == 0;
  const bool i8 = ep.out_mode == OUT_I8_ACT;
  if ((g.Cp % 32) != 0 || g.row_bytes != 0 || g.dw || (!i8 && ep.residual) || ep.pool ||
      !(nopad || (g.KH <= 32 && g.KW <= 32)) || first_block < 0)
    return arg_error("conv_group_layer: not eligible (few-channel input, depthwise, fused pool)");
  // the 8-wavefront configuration with the tile the usual choice would take (int8 output: always 32 channels)
  const int usual = choose_wave_cfg(g);
  int cfg = i8 || (usual >= 4 && usual <= 6) || g.OC <= 32 ? 4 : 0;
  const int mode = (g.KH == 1 && g.KW == 1 && g.SH == 1 && g.SW == 1 && nopad && g.OH == g.H && g.OW == g.W)
                       ? WAVE_IDENT : nopad ? WAVE_NOPAD : WAVE_PAD;
  // int8 entries with fewer than two chunks per wavefront after the split: eight wavefronts side by side, unsplit
  static const WaveCfg kUnsplit8 = {1, 2, 1, 8, 2};
  const bool unsplit = i8 && g.K / 32 < 16;
  const WaveCfg& c = unsplit ? kUnsplit8 : kWaveCfgs[cfg];
  if (unsplit) cfg = 8;   // any code but 4: see group8_layer
  const int64_t nb = wave_cfg_blocks(c, g);
  if (nb > 65536) return arg_error("conv_group_layer: not eligible (a layer that fills the chip by itself)");
  g.octiles = (g.OC + 32 * c.tm - 1) / (32 * c.tm);
  g.div_octiles = make_fastdiv((uint32_t)g.octiles);
  SeqLayer& L = reinterpret_cast<SeqLayer*>(table)[index];
  memset(&L, 0, sizeof(L));
  L.px_per_share = first_block;
  L.ptiles = (int)nb;
  L.kernel = cfg * 3 + (mode == WAVE_IDENT ? 0 : mode == WAVE_NOPAD ? 1 : 2);
  L.xp = xp;
  L.wf = wp;
  L.out = out;
  L.g = g;
  L.ep = ep;
  if (blocks) *blocks = (int)nb;
  return CVMHIP_OK;
}
int conv_group_launch(const void* dev_table, int nlayers, int total_blocks, int out_is_i8, double ops, double bytes, hipStream_t s) {
  if (!dev_table || nlayers < 1 || total_blocks < 1 || ((uintptr_t)dev_table & 15)) return arg_error("conv_group_launch");
  char desc[64];
  snprintf(desc, sizeof(desc), "%d independent convolutions in one launch, grid %d%s", nlayers, total_blocks, out_is_i8 ? " i8" : " i32");
  KernelTimer timer("k_conv_group", ops, s, bytes, desc);
  if (out_is_i8) k_conv_group8<<<(unsigned)total_blocks, 512, 0, s>>>(reinterpret_cast<const SeqLayer*>(dev_table), nlayers);
  else k_conv_group<<<(unsigned)total_blocks, 512, 0, s>>>(reinterpret_cast<const SeqLayer*>(dev_table), nlayers);
  return check_launch("conv_group");
}

// ---- layer-sequence launch: host side
size_t conv_seq_layer_bytes() { return sizeof(SeqLayer); }
int conv_seq_shares() { return SEQ_SHARES; }
size_t conv_seq_sync_bytes() { return (SEQ_SHARES + 1) * SEQ_SYNC_WORDS * sizeof(unsigned); }

// Fills entry `index` of a host copy of the table.  CVMHIP_ERR_ARG with "not eligible" when this convolution
// cannot be one layer of a sequence (the caller then launches it on its own).
int conv_seq_layer(void* table, int index, const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep_in) {
  Epilogue ep;
  const int prc = conv_prepare(xp, wp, out, g, ep_in, ep);
  if (prc) return prc;
  const bool nopad = g.PH == 0 && g.PW == 0;
  if ((g.Cp % 32) != 0 || g.row_bytes != 0 || g.dw || ep.out_mode != OUT_I8_ACT || ep.pool || !(nopad || (g.KH <= 32 && g.KW <= 32)))
    return arg_error("conv_seq_layer: not eligible (few-channel input, depthwise or int32 output)");
  // results are stored through a buffer descriptor with 32-bit offsets
  if (act_bytes(g.P, ep.out_cp) > INT32_MAX) return arg_error("conv_seq_layer: not eligible (output tensor of 2 GiB or more)");
  // the sequence kernel carries code for short chains without multiplications only
  for (const DevChain* c : {&ep.chain, &ep.chain2}) {
    if (c->count > SEQ_MAX_STAGES) return arg_error("conv_seq_layer: not eligible (a requantisation chain of more than two stages)");
    for (int t = 0; t < c->count; ++t)
      if (c->st[t].mul != 1) return arg_error("conv_seq_layer: not eligible (a requantisation chain that multiplies)");
  }
  const ConvTuning tune = t_conv_tuning;
  // a layer that fills the chip several times over is faster as a launch of the large-tile kernel than as a layer of a
  // sequence (whose tile is the wavefront kernel's); a run of layers ends there
  if (tune.kernel == CONV_KERNEL_AUTO && tune.wave_cfg < 0 && choose_big_cfg(g) >= 0)
    return arg_error("conv_seq_layer: not eligible (a layer for the large-tile kernel)");
  SeqLayer& L = reinterpret_cast<SeqLayer*>(table)[index];
  memset(&L, 0, sizeof(L));
  // whole images per share: as many XCDs as divide the batch (8, 4, 2 or 1)
  int shares = SEQ_SHARES;
  while (g.N % shares != 0) shares >>= 1;
  L.shares = shares;
  L.px_per_share = (int)(g.P / shares);
  // the configuration is chosen for one share on the 32 compute units of its XCD
  ConvGeom share = g;
  share.P = L.px_per_share;
  int cfg = choose_wave_cfg(share, SEQ_WG_PER_SHARE);
  if (tune.wave_cfg >= 0 && tune.wave_cfg <= 6) cfg = tune.wave_cfg;
  if (index < 64 && tune.seq_layer_cfg[index] >= 0 && tune.seq_layer_cfg[index] <= 6) cfg = tune.seq_layer_cfg[index];
  if (cfg > 6) cfg = 3;
  const int mode = (g.KH == 1 && g.KW == 1 && g.SH == 1 && g.SW == 1 && nopad && g.OH == g.H && g.OW == g.W)
                       ? WAVE_IDENT : nopad ? WAVE_NOPAD : WAVE_PAD;
  const WaveCfg& c = kWaveCfgs[cfg];
  const int bm = 32 * c.tm, bn = 32 * c.tn * (c.nw / c.ksplit);
  g.octiles = (g.OC + bm - 1) / bm;
  g.div_octiles = make_fastdiv((uint32_t)g.octiles);
  // a share begins at a multiple of px_per_share, which need not be a multiple of 32: its first pixel block
  // may start up to 31 pixels early (those pixels are computed and not stored)
  int ptiles = 0;
  for (int x = 0; x < shares; ++x) {
    const int lead = (x * L.px_per_share) & 31;
    const int t = (lead + L.px_per_share + bn - 1) / bn;
    ptiles = t > ptiles ? t : ptiles;
  }
  L.ptiles = ptiles;
  L.kernel = cfg * 3 + (mode == WAVE_IDENT ? 0 : mode == WAVE_NOPAD ? 1 : 2);
  L.xp = xp;
  L.wf = wp;
  L.out = out;
  L.g = g;
  L.ep = ep;
  return CVMHIP_OK;
}

int conv_seq_layer_config(const void* table, int index) {
  return reinterpret_cast<const SeqLayer*>(table)[index].kernel / 3;
}

int conv_seq_layer_chain(const void* table, int index) {
  const SeqLayer& l = reinterpret_cast<const SeqLayer*>(table)[index];
  return l.chain + 16 * l.join_next;
}

// ---- chains: 1x1 layers computed by the wavefront that holds their input (conv_chain_tail)
static bool ranges_overlap(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes) {
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}
// Layer `f` of the table can follow layer `prev` inside a chain that began with layer `a`: a 1x1 convolution with stride
// 1 and no padding over prev's output, pixel for pixel, whole 32-channel tiles on both sides.
static bool chain_follower(const SeqLayer& a, const SeqLayer& prev, const SeqLayer& f) {
  if (f.kernel % 3 != 0 || f.xp != prev.out || f.g.P != a.g.P || f.shares != a.shares || f.px_per_share != a.px_per_share) return false;
  if (f.g.Cp != prev.g.OC || prev.ep.out_cp != prev.g.OC || (f.g.OC & 31) != 0 || f.ep.out_cp != f.g.OC) return false;
  if (f.g.Kp != ((f.g.Cp + 63) & ~63)) return false;   // the filter's chunks are the input's 32-channel tiles
  if (f.ep.bias && !f.ep.bias_vec) return false;
  return true;
}
static int chain_followers(const SeqLayer* L, int i, int count) {
  const SeqLayer& a = L[i];
  if (i + 1 >= count || a.g.OC != 64 || a.ep.out_cp != 64 || a.ep.residual || a.g.octiles < 1) return 0;
  const SeqLayer& b = L[i + 1];
  if (!chain_follower(a, a, b)) return 0;
  const int64_t a_in = act_bytes((int64_t)a.g.N * a.g.H * a.g.W, a.g.Cp), a_out = act_bytes(a.g.P, 64), b_out = act_bytes(a.g.P, b.g.OC);
  // While one wavefront stores its pixels of A, B and C, others still read A's input around theirs, and B's residual at
  // theirs: no output may lie over either, nor over another output.  (The residual itself may be B's output tensor:
  // a block of it is read and written by the same wavefront, in that order.)
  if (ranges_overlap(a.out, a_out, a.xp, a_in) || ranges_overlap(b.out, b_out, a.xp, a_in) || ranges_overlap(a.out, a_out, b.out, b_out)) return 0;
  if (b.ep.residual) {
    if (b.ep.residual != b.out && ranges_overlap(b.out, b_out, b.ep.residual, b_out)) return 0;
    if (ranges_overlap(a.out, a_out, b.ep.residual, b_out)) return 0;
  }
  // the filters are copied to the workgroup's 128 KiB LDS block and the biases to 512 words beside it
  auto filter = [](const SeqLayer& l) { return (int64_t)(l.g.OC / 32) * (l.g.Kp / 32 + 1) * 1024; };
  if (filter(a) + filter(b) > 131072 || b.g.OC > 512) return 0;
  if (i + 2 >= count) return 1;
  const SeqLayer& c = L[i + 2];
  if (filter(a) + filter(b) + filter(c) > 131072 || b.g.OC + c.g.OC > 512) return 1;
  if (!chain_follower(a, b, c) || c.ep.residual || (c.g.OC != 64 && c.g.OC != 128)) return 1;
  const int64_t c_out = act_bytes(a.g.P, c.g.OC);
  if (ranges_overlap(c.out, c_out, a.xp, a_in) || ranges_overlap(c.out, c_out, a.out, a_out) || ranges_overlap(c.out, c_out, b.out, b_out)) return 1;
  if (b.ep.residual && ranges_overlap(c.out, c_out, b.ep.residual, b_out)) return 1;
  return 2;
}
// What a layer (with the chain behind it, n followers) reads and writes, as address ranges.
struct Footprint {
  const void* r[2]; int64_t rb[2]; int nr;
  const void* w[3]; int64_t wb[3]; int nw;
};
static Footprint footprint(const SeqLayer* L, int i) {
  Footprint f{};
  const SeqLayer& a = L[i];
  f.r[f.nr] = a.xp; f.rb[f.nr++] = act_bytes((int64_t)a.g.N * a.g.H * a.g.W, a.g.Cp);
  for (int k = 0; k <= a.chain; ++k) {
    const SeqLayer& l = L[i + k];
    f.w[f.nw] = l.out; f.wb[f.nw++] = act_bytes(l.g.P, l.ep.out_cp);
    if (l.ep.residual && f.nr < 2) { f.r[f.nr] = l.ep.residual; f.rb[f.nr++] = act_bytes(l.g.P, l.ep.out_cp); }
  }
  return f;
}
static bool independent(const Footprint& p, const Footprint& q) {
  for (int i = 0; i < p.nw; ++i) {
    for (int j = 0; j < q.nr; ++j) if (ranges_overlap(p.w[i], p.wb[i], q.r[j], q.rb[j])) return false;
    for (int j = 0; j < q.nw; ++j) if (ranges_overlap(p.w[i], p.wb[i], q.w[j], q.wb[j])) return false;
  }
  for (int i = 0; i < q.nw; ++i)
    for (int j = 0; j < p.nr; ++j) if (ranges_overlap(q.w[i], q.wb[i], p.r[j], p.rb[j])) return false;
  return true;
}

// Links the chains of a finished table of `count` entries (after every conv_seq_layer call, before it is copied to the
// device); returns how many it found.  A layer whose configuration was forced is left as it is.
int conv_seq_link(void* table, int count) {
  const ConvTuning tune = t_conv_tuning;
  if (!tune.seq_chains || tune.wave_cfg >= 0 || tune.kernel != CONV_KERNEL_AUTO) return 0;
  SeqLayer* L = reinterpret_cast<SeqLayer*>(table);
  int linked = 0;
  for (int i = 0; i + 1 < count;) {
    int n = chain_followers(L, i, count);
    for (int k = 0; k <= n; ++k)
      if (i + k < 64 && tune.seq_layer_cfg[i + k] >= 0) n = 0;
    if (n == 0) { ++i; continue; }
    SeqLayer& a = L[i];
    a.chain = n;
    a.kernel = 7 * 3 + a.kernel % 3;
    a.g.octiles = 1;
    a.g.div_octiles = make_fastdiv(1u);
    int ptiles = 0;
    for (int x = 0; x < a.shares; ++x) {
      const int lead = (x * a.px_per_share) & 31;
      const int t = (lead + a.px_per_share + 31) / 32;   // a pixel block per wavefront
      ptiles = t > ptiles ? t : ptiles;
    }
    a.ptiles = ptiles;
    ++linked;
    i += n + 1;
  }
  // Two layers in a row of which the second neither reads what the first writes nor writes what the first touches (the
  // first 1x1 layer and the shortcut projection of a ResNet block) need no boundary between them: a workgroup that is
  // through with the first goes on to the second.  Pairs only -- a third layer would have to be independent of both.
  for (int i = 0; i < count;) {
    const int j = i + 1 + L[i].chain;
    if (j < count && L[i].chain == 0 && L[i].shares == L[j].shares && independent(footprint(L, i), footprint(L, j))) {
      L[i].join_next = 1;
      ++linked;
      i = j + 1 + L[j].chain;
    } else {
      i = j;
    }
  }
  return linked;
}

int conv_seq_launch(const void* dev_table, int nlayers, void* sync, double ops, double bytes, hipStream_t s) {
  if (!dev_table || nlayers < 1 || !sync || ((uintptr_t)dev_table & 15) || ((uintptr_t)sync & 255)) return arg_error("conv_seq_launch");
  char desc[64];
  snprintf(desc, sizeof(desc), "%d convolutions in one launch", nlayers);
  KernelTimer timer("k_conv_seq", ops, s, bytes, desc);
  const ConvTuning tune = t_conv_tuning;
  k_conv_seq<<<SEQ_SHARES * SEQ_WG_PER_SHARE, 512, 0, s>>>(reinterpret_cast<const SeqLayer*>(dev_table), nlayers,
                                                          reinterpret_cast<unsigned*>(sync), tune.seq_spin_limit, tune.seq_stamps,
                                                          tune.seq_stamp_layers);
  return check_launch("conv_seq");
}

}  // namespace cvmhip

using namespace cvmhip;

extern "C" {

int cvmhip_set_conv_tuning(int kernel, int wave_cfg, int tile_wm, int tile_wn) {
  if (kernel < CONV_KERNEL_AUTO || kernel > CONV_KERNEL_BIG) return arg_error("set_conv_tuning kernel");
  ConvTuning t = t_conv_tuning;
  t.kernel = kernel; t.wave_cfg = wave_cfg; t.tile_wm = tile_wm; t.tile_wn = tile_wn;
  set_conv_tuning(t);
  return CVMHIP_OK;
}

int cvmhip_set_seq_layer_config(int index, int config) {
  ConvTuning t = t_conv_tuning;
  if (index < 0) memset(t.seq_layer_cfg, -1, sizeof(t.seq_layer_cfg));   // all automatic again
  else if (index < 64 && config >= -1 && config < 127) t.seq_layer_cfg[index] = (signed char)config;
  else return arg_error("set_seq_layer_config");
  set_conv_tuning(t);
  return CVMHIP_OK;
}

int cvmhip_set_seq_stamps(void* stamps, int layers) {
  if (layers < 0 || (stamps && ((uintptr_t)stamps & 7))) return arg_error("set_seq_stamps");
#ifndef CVM_SEQ_STAMPS
  if (stamps) return arg_error("set_seq_stamps: this build has no time stamps (build with -DCVM_SEQ_STAMPS)");
#endif
  ConvTuning t = t_conv_tuning;
  t.seq_stamps = stamps && layers > 0 ? reinterpret_cast<unsigned long long*>(stamps) : nullptr;
  t.seq_stamp_layers = t.seq_stamps ? layers : 0;
  set_conv_tuning(t);
  return CVMHIP_OK;
}

int cvmhip_set_seq_tuning(int spin_limit) {
  if (spin_limit < 0) return arg_error("set_seq_tuning");
  ConvTuning t = t_conv_tuning;
  t.seq_spin_limit = spin_limit;
  set_conv_tuning(t);
  return CVMHIP_OK;
}

int cvmhip_set_seq_chains(int on) {
  ConvTuning t = t_conv_tuning;
  t.seq_chains = on != 0;
  set_conv_tuning(t);
  return CVMHIP_OK;
}

size_t cvmhip_conv2d_workspace_bytes(int n, int ic, int h, int w, int oc, int kh, int kw, int groups) {
  if (groups != 1) return 0;
  return packed_act_bytes((int64_t)n * h * w, ic) + packed_weight_bytes(oc, ic, kh, kw);
}

int cvmhip_conv2d(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                  int n, int ic, int h, int wd, int oc, int kh, int kw,
                  int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                  int groups, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !w || !y) return arg_error("conv2d null tensor");
  if (n < 1 || ic < 1 || h < 1 || wd < 1 || oc < 1 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
      pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1 || groups < 1 || ic % groups || oc % groups)
    return arg_error("conv2d attributes");
  const int oh = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  const int ow = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  if (h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1) return arg_error("conv2d kernel exceeds input");
  hipStream_t s = as_stream(stream);
  if (groups > 1) {
    const int64_t total = (int64_t)n * oc * oh * ow;
    k_conv_grouped<<<grid_for(total, 256, 1 << 20), 256, 0, s>>>(x, w, bias, y, total, ic, h, wd, oc, oh, ow, kh, kw,
                                                               stride_h, stride_w, pad_h, pad_w, dil_h, dil_w,
                                                               ic / groups, oc / groups);
    return check_launch("conv_grouped");
  }
  const size_t need = cvmhip_conv2d_workspace_bytes(n, ic, h, wd, oc, kh, kw, 1);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return arg_error("conv2d workspace");
  int8_t* xp = reinterpret_cast<int8_t*>(workspace);
  int8_t* wp = xp + packed_act_bytes((int64_t)n * h * wd, ic);
  int rc = pack_activations(x, xp, n, ic, h * wd, s);
  if (rc) return rc;
  rc = pack_weights(w, wp, oc, ic, kh, kw, s);
  if (rc) return rc;
  ConvGeom g = {};
  g.N = n; g.H = h; g.W = wd; g.Cp = pad_channels(ic); g.C = ic;
  g.OC = oc; g.OH = oh; g.OW = ow;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = pad_h; g.PW = pad_w; g.DH = dil_h; g.DW = dil_w;
  Epilogue ep = {};
  ep.bias = bias;
  ep.out_mode = OUT_I32_NCHW;
  return conv_igemm(xp, wp, y, g, ep, s);
}

size_t cvmhip_dense_workspace_bytes(int m, int k, int n) {
  return packed_act_bytes(m, k) + packed_weight_bytes(n, k, 1, 1);
}

int cvmhip_dense(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                 int m, int k, int n, int operand_bits,
                 void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !w || !y || m < 1 || k < 1 || n < 1) return arg_error("dense");
  hipStream_t s = as_stream(stream);
  if (operand_bits > 8) {
    const int64_t total = (int64_t)((m + DENSE_MB - 1) / DENSE_MB) * n;
    k_dense_i32<<<grid_for(total * 64, 256, 1 << 20), 256, 0, s>>>(x, w, bias, y, m, k, n);
    return check_launch("dense_i32");
  }
  const size_t need = cvmhip_dense_workspace_bytes(m, k, n);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return arg_error("dense workspace");
  // x[m][k] is already "NHWC" with one pixel per row; the filter is OC x K x 1 x 1
  int8_t* xp = reinterpret_cast<int8_t*>(workspace);
  int8_t* wp = xp + packed_act_bytes(m, k);
  int rc = pack_activations(x, xp, m, k, 1, s);
  if (rc) return rc;
  rc = pack_weights(w, wp, n, k, 1, 1, s);
  if (rc) return rc;
  ConvGeom g = {};
  g.N = m; g.H = 1; g.W = 1; g.Cp = pad_channels(k); g.C = k;
  g.OC = n; g.OH = 1; g.OW = 1;
  g.KH = g.KW = g.SH = g.SW = g.DH = g.DW = 1;
  Epilogue ep = {};
  ep.bias = bias;
  ep.out_mode = OUT_I32_NCHW;
  return conv_igemm(xp, wp, y, g, ep, s);
}

size_t cvmhip_packed_weight_bytes(int oc, int ic, int kh, int kw) { return packed_weight_bytes(oc, ic, kh, kw); }

size_t cvmhip_packed_act_bytes(int64_t npix, int channels) { return packed_act_bytes(npix, channels); }

int cvmhip_pack_weights(const int32_t* w, void* wp, int oc, int ic, int kh, int kw, void* stream) {
  if (!w || !wp || oc < 1 || ic < 1 || kh < 1 || kw < 1 || ((uintptr_t)wp & 15)) return arg_error("pack_weights");
  return pack_weights(w, reinterpret_cast<int8_t*>(wp), oc, ic, kh, kw, as_stream(stream));
}

int cvmhip_conv2d_packed(const int32_t* x, const void* wp, const int32_t* bias, int32_t* y,
                         int n, int ic, int h, int wd, int oc, int kh, int kw,
                         int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                         void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !wp || !y) return arg_error("conv2d_packed null tensor");
  if (n < 1 || ic < 1 || h < 1 || wd < 1 || oc < 1 || kh < 1 || kw < 1 || stride_h < 1 || stride_w < 1 ||
      pad_h < 0 || pad_w < 0 || dil_h < 1 || dil_w < 1)
    return arg_error("conv2d_packed attributes");
  if (h + 2 * pad_h < dil_h * (kh - 1) + 1 || wd + 2 * pad_w < dil_w * (kw - 1) + 1)
    return arg_error("conv2d_packed kernel exceeds input");
  const size_t need = packed_act_bytes((int64_t)n * h * wd, ic);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return arg_error("conv2d_packed workspace");
  hipStream_t s = as_stream(stream);
  int8_t* xp = reinterpret_cast<int8_t*>(workspace);
  int rc = pack_activations(x, xp, n, ic, h * wd, s);
  if (rc) return rc;
  ConvGeom g = {};
  g.N = n; g.H = h; g.W = wd; g.Cp = pad_channels(ic); g.C = ic;
  g.OC = oc;
  g.OH = (h + 2 * pad_h - (dil_h * (kh - 1) + 1)) / stride_h + 1;
  g.OW = (wd + 2 * pad_w - (dil_w * (kw - 1) + 1)) / stride_w + 1;
  g.KH = kh; g.KW = kw; g.SH = stride_h; g.SW = stride_w; g.PH = pad_h; g.PW = pad_w; g.DH = dil_h; g.DW = dil_w;
  Epilogue ep = {};
  ep.bias = bias;
  ep.out_mode = OUT_I32_NCHW;
  return conv_igemm(xp, reinterpret_cast<const int8_t*>(wp), y, g, ep, s);
}

}  // extern "C"
