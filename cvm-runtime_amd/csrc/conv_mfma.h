// Internal interface of the int8 implicit-GEMM convolution (conv_mfma.hip),
// shared by the operator-level C ABI and the fused graph executor.
#ifndef CVM_CONV_MFMA_H_
#define CVM_CONV_MFMA_H_

#include "hip_common.h"

namespace cvmhip {

enum { OUT_I32_NCHW = 0, OUT_I8_NHWC = 1 };

struct ConvGeom {
  int N, H, W, Cp;         // input: int8 NHWC, channels padded to Cp
  int C;                   // true channel count (0 = unknown, only used to count algorithmic work)
  int OC, OH, OW;          // output extent
  int KH, KW, SH, SW, PH, PW, DH, DW;
  int taps, K, Kp;         // filled by conv_igemm: KH*KW, taps*Cp, K rounded up to 64
  int64_t P;               // filled by conv_igemm: N*OH*OW
  int adv_c, adv_tap, adv_r, adv_s;  // filled by conv_igemm: cursor advance of one K step (channel, tap, filter row/column)
};

// What happens to an accumulator before it is stored:
//   v = chain(acc + bias[oc]);  if (residual) v = chain2(v + residual[p][oc]);
struct Epilogue {
  const int32_t* bias;     // device pointer or nullptr
  int bias_vec;            // set by conv_igemm: bias is 16-byte aligned
  DevChain chain;
  const int8_t* residual;  // int8 NHWC with pitch out_cp, or nullptr
  DevChain chain2;
  int out_mode;            // OUT_I32_NCHW or OUT_I8_NHWC
  int out_cp;              // channel pitch of int8 NHWC output / residual (multiple of 4, >= OC)
};

int pad_channels(int c);
size_t packed_act_bytes(int64_t npix, int c);
void weight_dims(int oc, int ic, int kh, int kw, int* ocp, int* kp);
size_t packed_weight_bytes(int oc, int ic, int kh, int kw);

int pack_activations(const int32_t* x, int8_t* xp, int n, int c, int hw, hipStream_t s);
int unpack_activations(const int8_t* xp, int32_t* x, int n, int c, int hw, hipStream_t s);
int pack_weights(const int32_t* w, int8_t* wp, int oc, int ic, int kh, int kw, hipStream_t s);
int conv_igemm(const int8_t* xp, const int8_t* wp, void* out, ConvGeom g, const Epilogue& ep, hipStream_t s);

}  // namespace cvmhip
#endif
