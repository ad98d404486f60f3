// conv2d / dense on gfx950 as an exact int8 x int8 -> int32 implicit GEMM.
//
//   D[oc][px] = sum_k Wp[oc][k] * Xcol[px][k],   k = (kh, kw, c),  px = (n, oh, ow)
//
// Data layout
//   Xp : int8 NHWC activations, channels padded to Cp (4, 8 or a multiple of 16)
//   Wp : int8 [OCp][Kp] filter rows, k ordered (kh, kw, c) with c padded to Cp,
//        Kp = K rounded up to 64, OCp = OC rounded up to 128; padding is zero
//   D  : int32 NCHW (the operator contract) or int8 NHWC (fused requantised output)
//
// One workgroup = 4 wavefronts (2 x 2) and computes a (64*WM) x (64*WN) tile of
// D with v_mfma_i32_32x32x32_i8.  Each K step stages a KS-byte slab (64 or 128)
// of both operands in LDS (row pitch KS+16 bytes, so the 16-byte MFMA operand
// reads of 8 consecutive lanes hit disjoint banks); the im2col addressing
// happens while the slab is fetched, so no column buffer ever exists in HBM.
// Global fetches run two K steps ahead of the MFMAs (registers hold step t+1
// and t+2 while LDS holds t and t+1), with one barrier per step.  The int8
// epilogue transposes the tile through LDS so that every lane writes 16
// contiguous output bytes.
#include <stdlib.h>

#include <type_traits>

#include "conv_mfma.h"

namespace cvmhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ int4 zero4() { return make_int4(0, 0, 0, 0); }

// Source of every out-of-image (padding) granule: loads stay unconditional and
// the data needs no fix-up before it goes to LDS, so nothing but the loads
// themselves sits between a fetch and the matrix instructions of that K step.
__device__ __attribute__((aligned(16))) int g_zero_granule[4] = {0, 0, 0, 0};  // never written

// Fetch the 16 consecutive k-bytes of one im2col row that start at filter tap
// (r, s), channel c0.  G = bytes that are contiguous in memory for one filter
// tap: 16 when Cp % 16 == 0, else Cp itself (4 or 8) and the chunk spans 16/G taps.
template <int G>
__device__ __forceinline__ int4 fetch_act(const int8_t* __restrict__ xp, const ConvGeom& g, bool row_ok, int img_off,
                                          int ih0, int iw0, int tap, int r, int s, int c0) {
  const int8_t* zero = reinterpret_cast<const int8_t*>(g_zero_granule);
  if (G == 16) {
    const int ih = ih0 + r * g.DH, iw = iw0 + s * g.DW;
    const bool ok = row_ok && tap < g.taps && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
    const int8_t* src = ok ? xp + (img_off + (ih * g.W + iw) * g.Cp + c0) : zero;
    return *reinterpret_cast<const int4*>(src);
  } else {
    int v[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16 / G; ++j) {
      const int t = tap + j;
      const int rr = t / g.KW, ss = t - rr * g.KW;
      const int ih = ih0 + rr * g.DH, iw = iw0 + ss * g.DW;
      const bool ok = row_ok && t < g.taps && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
      const int8_t* src = ok ? xp + (img_off + (ih * g.W + iw) * g.Cp) : zero;
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

// clamp(v, lo, hi) for lo <= hi in one instruction
__device__ __forceinline__ int32_t clamp3(int32_t v, int32_t lo, int32_t hi) {
  int32_t r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
  return r;
}

template <int WM, int WN, int G, int KS, int OUT>
__global__ void __launch_bounds__(256)
k_conv_igemm(const int8_t* __restrict__ xp, const int8_t* __restrict__ wp, void* __restrict__ out,
             const ConvGeom g, const Epilogue ep) {
  constexpr int BM = 64 * WM;        // output channels per workgroup
  constexpr int BN = 64 * WN;        // output pixels per workgroup
  constexpr int LDK = KS + 16;       // LDS row pitch in bytes
  constexpr int CPR = KS / 16;       // 16-byte chunks per row and K step
  constexpr int RPP = 256 / CPR;     // rows one pass of the workgroup covers
  constexpr int NA = BM / RPP;       // filter chunks per thread and K step
  constexpr int NB = BN / RPP;       // activation chunks per thread and K step
  constexpr int OPITCH = BM + 4;     // pitch of the transposed int8 output tile (odd number of dwords)
  static_assert(BN * OPITCH <= 2 * BM * LDK, "output tile must fit the filter staging area");
  __shared__ __attribute__((aligned(16))) int8_t sA[2 * BM * LDK];
  __shared__ __attribute__((aligned(16))) int8_t sB[2 * BN * LDK];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // XCD-aware tile order: workgroups are dealt round-robin to the 8 XCDs, so
  // give each XCD a contiguous run of tiles (neighbouring tiles share the
  // activation slab in that XCD's L2).
  int pid = blockIdx.x;
  const int nb = gridDim.x;
  if ((nb & 7) == 0) pid = (pid & 7) * (nb >> 3) + (pid >> 3);
  const int oc_tiles = (g.OC + BM - 1) / BM;
  const int oc0 = (pid % oc_tiles) * BM;
  const int64_t px0 = (int64_t)(pid / oc_tiles) * BN;

  // ---- per-thread fetch assignment: chunk column kc, rows frow + RPP*i
  const int kc = tid % CPR;
  const int frow = tid / CPR;
  const int OHW = g.OH * g.OW;
  bool row_ok[NB];
  int img_off[NB], ih0[NB], iw0[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int64_t p = px0 + frow + RPP * i;
    row_ok[i] = p < g.P;
    const int pp = row_ok[i] ? (int)p : 0;
    const int n = pp / OHW;
    const int rem = pp - n * OHW;
    const int oh = rem / g.OW, ow = rem - oh * g.OW;
    img_off[i] = n * g.H * g.W * g.Cp;
    ih0[i] = oh * g.SH - g.PH;
    iw0[i] = ow * g.SW - g.PW;
  }
  const int8_t* wbase = wp + (int64_t)(oc0 + frow) * g.Kp + kc * 16;

  // position of this thread's chunk inside the (tap, channel) space
  int tap = (kc * 16) / g.Cp, c0 = kc * 16 - tap * g.Cp;
  int r = tap / g.KW, s = tap - r * g.KW;
  int kbyte = 0;

  // Accumulator element e of lane l in a 32x32 tile is row (e/4)*8 + (l/32)*4 + e%4
  // (output channel), column l%32 (pixel).  Accumulators start at the bias of
  // their channel, so the epilogue has no bias pass.
  const int lrow = lane & 31;
  const int lgrp = lane >> 5;
  v16i acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    v16i b;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int oc = oc0 + (wm * WM + i) * 32 + q * 8 + lgrp * 4;
      int4 bv = zero4();
      if (ep.bias) {
        if (ep.bias_vec && oc + 3 < g.OC) {
          bv = *reinterpret_cast<const int4*>(ep.bias + oc);
        } else {
          if (oc < g.OC) bv.x = ep.bias[oc];
          if (oc + 1 < g.OC) bv.y = ep.bias[oc + 1];
          if (oc + 2 < g.OC) bv.z = ep.bias[oc + 2];
          if (oc + 3 < g.OC) bv.w = ep.bias[oc + 3];
        }
      }
      b[q * 4] = bv.x; b[q * 4 + 1] = bv.y; b[q * 4 + 2] = bv.z; b[q * 4 + 3] = bv.w;
    }
#pragma unroll
    for (int j = 0; j < WN; ++j) acc[i][j] = b;
  }

  // One K step of operands held in registers as a single SSA vector value
  // (chunks 0..NA-1 filter, NA..NA+NB-1 activations); two of them are in flight.
  typedef int regs_t __attribute__((ext_vector_type(4 * (NA + NB))));
  const int nk = g.Kp / KS;

  // loads the next K step and advances the (tap, channel) cursor
  auto fetch = [&]() -> regs_t {
    regs_t R;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int4 v = *reinterpret_cast<const int4*>(wbase + (int64_t)(RPP * i) * g.Kp + kbyte);
      R[4 * i] = v.x; R[4 * i + 1] = v.y; R[4 * i + 2] = v.z; R[4 * i + 3] = v.w;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int4 v = fetch_act<G>(xp, g, row_ok[i], img_off[i], ih0[i], iw0[i], tap, r, s, c0);
      R[4 * (NA + i)] = v.x; R[4 * (NA + i) + 1] = v.y; R[4 * (NA + i) + 2] = v.z; R[4 * (NA + i) + 3] = v.w;
    }
    kbyte += KS;
    if (G == 16) {
      // advance the cursor by KS bytes without a loop (lanes sit at different chunks)
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
      *reinterpret_cast<int4*>(&sA[(buf * BM + frow + RPP * i) * LDK + kc * 16]) =
          make_int4(R[4 * i], R[4 * i + 1], R[4 * i + 2], R[4 * i + 3]);
#pragma unroll
    for (int i = 0; i < NB; ++i)
      *reinterpret_cast<int4*>(&sB[(buf * BN + frow + RPP * i) * LDK + kc * 16]) =
          make_int4(R[4 * (NA + i)], R[4 * (NA + i) + 1], R[4 * (NA + i) + 2], R[4 * (NA + i) + 3]);
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int ks = 0; ks < KS / 32; ++ks) {
      v4i a[WM], b[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[i] = *reinterpret_cast<const v4i*>(&sA[(buf * BM + (wm * WM + i) * 32 + lrow) * LDK + ks * 32 + lgrp * 16]);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j] = *reinterpret_cast<const v4i*>(&sB[(buf * BN + (wn * WN + j) * 32 + lrow) * LDK + ks * 32 + lgrp * 16]);
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
  // past the end reads valid memory (filter rows have slack behind them, taps
  // past the filter read the zero granule) and is never consumed -- because a conditional
  // fetch makes the compiler wait for all outstanding loads at the join.
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

  // ---- epilogue: v = chain(acc); if (residual) v = chain2(v + residual).
  // A chain runs stage by stage over all accumulators of the thread: the stage
  // parameters are wave-uniform, so each stage costs four vector instructions
  // per value (one for a pure clamp).
  auto run_chain = [&](const DevChain& c) __attribute__((always_inline)) {
    // the stages are copied to scalar registers first: indexing the kernel
    // argument with the loop counter would move it to private memory
    const DevStage q0 = c.st[0], q1 = c.st[1], q2 = c.st[2], q3 = c.st[3];
#pragma unroll 1
    for (int t = 0; t < c.count; ++t) {
      DevStage st;
      st.lo = t == 0 ? q0.lo : t == 1 ? q1.lo : t == 2 ? q2.lo : q3.lo;
      st.hi = t == 0 ? q0.hi : t == 1 ? q1.hi : t == 2 ? q2.hi : q3.hi;
      st.s1 = t == 0 ? q0.s1 : t == 1 ? q1.s1 : t == 2 ? q2.s1 : q3.s1;
      st.add = t == 0 ? q0.add : t == 1 ? q1.add : t == 2 ? q2.add : q3.add;
      st.s2 = t == 0 ? q0.s2 : t == 1 ? q1.s2 : t == 2 ? q2.s2 : q3.s2;
      if ((st.s1 | st.add | st.s2) == 0) {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = clamp3(acc[i][j][e], st.lo, st.hi);
      } else {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
              acc[i][j][e] = wadd(clamp3(acc[i][j][e], st.lo, st.hi) >> st.s1, st.add) >> st.s2;
      }
    }
  };
  if (ep.residual) {
    // one dword = the residual of 4 consecutive channels; loads are issued before the first chain runs
    uint32_t rp[WM][WN][4];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int64_t p = px0 + (wn * WN + j) * 32 + lrow;
      const int8_t* res = ep.residual + (p < g.P ? p : 0) * ep.out_cp;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int oc = oc0 + (wm * WM + i) * 32 + q * 8 + lgrp * 4;
          rp[i][j][q] = *reinterpret_cast<const uint32_t*>(res + (oc < ep.out_cp ? oc : 0));
        }
    }
    run_chain(ep.chain);
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          acc[i][j][e] = wadd(acc[i][j][e], (int32_t)(int8_t)(rp[i][j][e >> 2] >> (8 * (e & 3))));
    run_chain(ep.chain2);
  } else {
    run_chain(ep.chain);
  }

  if (OUT == OUT_I32_NCHW) {
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int64_t p = px0 + (wn * WN + j) * 32 + lrow;
      if (p >= g.P) continue;
      const int n = (int)p / OHW;
      const int rem = (int)p - n * OHW;
      int32_t* y32 = reinterpret_cast<int32_t*>(out) + (int64_t)n * g.OC * OHW + rem;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int oc = oc0 + (wm * WM + i) * 32 + (e >> 2) * 8 + lgrp * 4 + (e & 3);
          if (oc < g.OC) y32[(int64_t)oc * OHW] = acc[i][j][e];
        }
    }
  } else {
    // int8 NHWC: transpose the tile through LDS (the filter staging area is free
    // after the last barrier of the K loop) so that global stores are 16 contiguous bytes per thread
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int pl = (wn * WN + j) * 32 + lrow;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ol = (wm * WM + i) * 32 + q * 8 + lgrp * 4;
          const uint32_t lo2 = __builtin_amdgcn_perm((uint32_t)acc[i][j][q * 4 + 1], (uint32_t)acc[i][j][q * 4], 0x0c0c0400u);
          const uint32_t hi2 = __builtin_amdgcn_perm((uint32_t)acc[i][j][q * 4 + 3], (uint32_t)acc[i][j][q * 4 + 2], 0x0c0c0400u);
          *reinterpret_cast<uint32_t*>(&sA[pl * OPITCH + ol]) = __builtin_amdgcn_perm(hi2, lo2, 0x05040100u);
        }
    }
    __syncthreads();
    constexpr int CH = BM / 16;
    int8_t* y8 = reinterpret_cast<int8_t*>(out);
#pragma unroll
    for (int id = tid; id < BN * CH; id += 256) {
      const int pl = id / CH, c16 = id - pl * CH;
      const int64_t p = px0 + pl;
      const int oc = oc0 + c16 * 16;
      if (p >= g.P || oc >= ep.out_cp) continue;
      const uint32_t* src = reinterpret_cast<const uint32_t*>(&sA[pl * OPITCH + c16 * 16]);
      uint32_t d[4] = {src[0], src[1], src[2], src[3]};
      if (oc + 16 > g.OC) {
        // padding channels of the NHWC tensor stay zero whatever the chain maps 0 to
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int keep = g.OC - (oc + 4 * k);
          d[k] = keep >= 4 ? d[k] : (keep <= 0 ? 0u : d[k] & ((1u << (8 * keep)) - 1u));
        }
      }
      int8_t* dst = y8 + p * ep.out_cp + oc;
      if (oc + 16 <= ep.out_cp && (ep.out_cp & 15) == 0) {
        *reinterpret_cast<int4*>(dst) = make_int4(d[0], d[1], d[2], d[3]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (oc + k * 4 < ep.out_cp) reinterpret_cast<uint32_t*>(dst)[k] = d[k];
      }
    }
  }
}

constexpr int KSTEP = 64;  // granularity the packed filter rows are padded to

// ---------------------------------------------------------------- packing
// int32 NCHW -> int8 NHWC (channels padded to cp with zeros); narrowing is
// static_cast<int8_t>, the reference's own (ops.cc:234).
__global__ void __launch_bounds__(256) k_pack_nhwc(const int32_t* __restrict__ x, int8_t* __restrict__ xp, int64_t total,
                                                   int c, int hw, int cp) {
  const int c4n = cp / 4;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int pix = (int)(i % hw);
    const int64_t t = i / hw;
    const int c4 = (int)(t % c4n);
    const int64_t n = t / c4n;
    uint32_t pack = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ch = c4 * 4 + j;
      const int32_t v = ch < c ? x[((int64_t)n * c + ch) * hw + pix] : 0;
      pack |= (uint32_t)(uint8_t)(int8_t)v << (8 * j);
    }
    *reinterpret_cast<uint32_t*>(xp + ((int64_t)n * hw + pix) * cp + c4 * 4) = pack;
  }
}

// int32 OIHW -> int8 [OCp][Kp], k = (r*KW + s)*Cp + c, zero padded
__global__ void __launch_bounds__(256) k_pack_weights(const int32_t* __restrict__ w, int8_t* __restrict__ wp, int64_t total,
                                                      int oc, int ic, int taps, int cp, int kp) {
  const int k4n = kp / 4;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int k4 = (int)(i % k4n);
    const int64_t o = i / k4n;
    const int k = k4 * 4;
    const int tap = k / cp, c = k - tap * cp;
    uint32_t pack = 0;
    if (o < oc && tap < taps) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int32_t v = (c + j < ic) ? w[((int64_t)o * ic + c + j) * taps + tap] : 0;
        pack |= (uint32_t)(uint8_t)(int8_t)v << (8 * j);
      }
    }
    *reinterpret_cast<uint32_t*>(wp + o * kp + k) = pack;
  }
}

// int8 NHWC (padded to cp) -> int32 NCHW
__global__ void __launch_bounds__(256) k_unpack_nchw(const int8_t* __restrict__ xp, int32_t* __restrict__ x, int64_t total,
                                                     int c, int hw, int cp) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int pix = (int)(i % hw);
    const int64_t t = i / hw;
    const int ch = (int)(t % c);
    const int64_t n = t / c;
    x[i] = xp[((int64_t)n * hw + pix) * cp + ch];
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

// dense on int32 operands without narrowing: one wavefront per output element.
__global__ void __launch_bounds__(256)
k_dense_i32(const int32_t* __restrict__ x, const int32_t* __restrict__ w, const int32_t* __restrict__ bias,
            int32_t* __restrict__ y, int64_t total, int k, int n) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t o = wave; o < total; o += nwaves) {
    const int64_t m = o / n;
    const int j = (int)(o - m * n);
    const int32_t* xr = x + m * k;
    const int32_t* wr = w + (int64_t)j * k;
    int32_t acc = 0;
    for (int t = lane; t < k; t += 64) acc = wadd(acc, wmul(xr[t], wr[t]));
    for (int d = 32; d >= 1; d >>= 1) acc = wadd(acc, __shfl_xor(acc, d, 64));
    if (lane == 0) y[o] = wadd(acc, bias ? bias[j] : 0);
  }
}

// ---------------------------------------------------------------- host side
int pad_channels(int c) {
  if (c <= 4) return 4;
  if (c <= 8) return 8;
  return (c + 15) / 16 * 16;
}

size_t packed_act_bytes(int64_t npix, int c) { return ((size_t)npix * pad_channels(c) + 255) / 256 * 256; }

void weight_dims(int oc, int ic, int kh, int kw, int* ocp, int* kp) {
  const int cp = pad_channels(ic);
  *kp = (kh * kw * cp + KSTEP - 1) / KSTEP * KSTEP;
  *ocp = (oc + 127) / 128 * 128;
}

size_t packed_weight_bytes(int oc, int ic, int kh, int kw) {
  int ocp, kp;
  weight_dims(oc, ic, kh, kw, &ocp, &kp);
  return ((size_t)ocp * kp + 512 + 255) / 256 * 256;  // 512: fetches run up to two K steps past the end
}

int pack_activations(const int32_t* x, int8_t* xp, int n, int c, int hw, hipStream_t s) {
  const int cp = pad_channels(c);
  const int64_t total = (int64_t)n * (cp / 4) * hw;
  if (total == 0) return CVMHIP_OK;
  KernelTimer timer("k_pack_nhwc", (double)n * c * hw * 5.0, s);  // bytes: 4 read + 1 written per element
  k_pack_nhwc<<<grid_for(total, 256), 256, 0, s>>>(x, xp, total, c, hw, cp);
  return check_launch("pack_nhwc");
}

int unpack_activations(const int8_t* xp, int32_t* x, int n, int c, int hw, hipStream_t s) {
  const int64_t total = (int64_t)n * c * hw;
  if (total == 0) return CVMHIP_OK;
  k_unpack_nchw<<<grid_for(total, 256), 256, 0, s>>>(xp, x, total, c, hw, pad_channels(c));
  return check_launch("unpack_nchw");
}

int pack_weights(const int32_t* w, int8_t* wp, int oc, int ic, int kh, int kw, hipStream_t s) {
  int ocp, kp;
  weight_dims(oc, ic, kh, kw, &ocp, &kp);
  const int64_t total = (int64_t)ocp * (kp / 4);
  k_pack_weights<<<grid_for(total, 256), 256, 0, s>>>(w, wp, total, oc, ic, kh * kw, pad_channels(ic), kp);
  return check_launch("pack_weights");
}

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

int conv_igemm(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep_in, hipStream_t s) {
  const Epilogue& ep0 = ep_in;
  if (g.N < 1 || g.H < 1 || g.W < 1 || g.OC < 1 || g.OH < 1 || g.OW < 1 || g.KH < 1 || g.KW < 1 || g.SH < 1 ||
      g.SW < 1 || g.DH < 1 || g.DW < 1 || g.PH < 0 || g.PW < 0)
    return arg_error("conv geometry");
  if (g.Cp != 4 && g.Cp != 8 && (g.Cp % 16) != 0) return arg_error("conv channel padding");
  if (((uintptr_t)xp | (uintptr_t)wp) & 15) return arg_error("conv operand alignment");
  if ((ep0.out_mode == OUT_I8_NHWC || ep0.residual) && (ep0.out_cp % 4 != 0 || ep0.out_cp < g.OC))
    return arg_error("conv int8 output layout");
  if (((uintptr_t)out | (uintptr_t)ep0.residual) & 3) return arg_error("conv output alignment");
  if (ep0.out_mode == OUT_I8_NHWC && (ep0.out_cp & 15) == 0 && ((uintptr_t)out & 15)) return arg_error("conv output alignment");
  g.taps = g.KH * g.KW;
  g.K = g.taps * g.Cp;
  g.Kp = (g.K + KSTEP - 1) / KSTEP * KSTEP;
  g.P = (int64_t)g.N * g.OH * g.OW;
  if ((int64_t)g.N * g.H * g.W * g.Cp > INT32_MAX || g.P > INT32_MAX) return arg_error("conv tensor too large");
  Epilogue ep = ep_in;
  ep.bias_vec = ep.bias != nullptr && ((uintptr_t)ep.bias & 15) == 0;
  const bool wide = (g.Kp % 128) == 0;
  const int gran = g.Cp >= 16 ? 16 : g.Cp;
  // Tile choice: the largest tile that still yields >= 2 workgroups per CU;
  // small layers fall back to smaller tiles to keep all 256 CUs busy.
  auto blocks = [&](int bm, int bn) { return (int64_t)((g.OC + bm - 1) / bm) * ((g.P + bn - 1) / bn); };
  int wm = g.OC > 64 ? 2 : 1, wn = 2;
  if (blocks(64 * wm, 64 * wn) < 512 && wn == 2) wn = 1;
  if (blocks(64 * wm, 64 * wn) < 512 && wm == 2) wm = 1;
  // tuning hook: CVM_HIP_TILE="wm,wn" forces a tile shape (read once)
  static const char* forced = getenv("CVM_HIP_TILE");
  if (forced && forced[0] >= '1' && forced[0] <= '2' && forced[1] == ',' && forced[2] >= '1' && forced[2] <= '2') {
    wm = forced[0] - '0';
    wn = forced[2] - '0';
  }
  const int64_t nb = blocks(64 * wm, 64 * wn);
  if (nb > 0x7fffffff) return arg_error("conv grid too large");
  const unsigned grid = (unsigned)nb;
  // algorithmic work of this launch: 2 * pixels * OC * (true channels * taps); padding not counted
  KernelTimer timer("k_conv_igemm", 2.0 * (double)g.P * g.OC * (double)g.taps * (double)(g.C ? g.C : g.Cp), s);
  const int ks = (wide && wm + wn < 4) ? 128 : 64;
  g.adv_c = ks % g.Cp;
  g.adv_tap = ks / g.Cp;
  g.adv_r = g.adv_tap / g.KW;
  g.adv_s = g.adv_tap % g.KW;
  if (ep.out_mode == OUT_I8_NHWC) launch_out<OUT_I8_NHWC>(wm, wn, gran, wide, grid, s, xp, wp, out, g, ep);
  else launch_out<OUT_I32_NCHW>(wm, wn, gran, wide, grid, s, xp, wp, out, g, ep);
  return check_launch("conv_igemm");
}

}  // namespace cvmhip

using namespace cvmhip;

extern "C" {

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
    const int64_t total = (int64_t)m * n;
    k_dense_i32<<<grid_for(total * 64, 256, 1 << 20), 256, 0, s>>>(x, w, bias, y, total, k, n);
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
