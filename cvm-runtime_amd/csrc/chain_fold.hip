// Host-side algebra on requantisation chains (no device code).
//
// cvmhip_fold_requant: the epilogue of a convolution is  v = chain(acc + bias[oc]);  if (residual) v = chain2(v + r).
// For the usual chains -- cvm_right_shift in its saturating regime, then clip / relu -- make_chain leaves one
// stage per chain,  (clamp(x, lo, hi) + 2^(b-1)) >> b,  i.e. three instructions per value (clamp, add, shift).  The
// add can be done once per channel instead of once per value: with T = 2^(b-1)
//     (clamp(x, lo, hi) + T) >> b  ==  clamp(x + T, lo + T, hi + T) >> b          whenever x + T does not wrap,
// and x + T = acc + (bias + T).  The same works one level up for the stage behind the residual add:
//     ((c1 + T1) >> b1) + T2  ==  (c1 + T1 + (T2 << b1)) >> b1,
// so chain2's rounding term T2 travels through the first shift into the bias as well, and chain2's clamp bounds
// move by T2.  "Does not wrap" is proven from the bias values themselves and a bound on |acc| (int8 x int8 products,
// a known number of terms); when the proof fails the function reports "not folded" and the caller keeps the
// original epilogue.  Clamp bounds that would leave the int32 range saturate: such a bound lies outside the proven
// range of the value, so it is never the active one.
#include <stdint.h>

#include <vector>

#include "hip_common.h"

using namespace cvmhip;

namespace {

int32_t sat_add(int32_t a, int64_t b) {
  const int64_t s = (int64_t)a + b;
  return s < INT32_MIN ? INT32_MIN : (s > INT32_MAX ? INT32_MAX : (int32_t)s);
}

// a stage that is clamp -> add -> shift and nothing else
bool plain_stage(const DevStage& s) { return s.mul == 1 && s.s1 == 0; }

bool to_public(const DevChain& c, cvmhip_chain* out) {
  out->count = c.count;
  for (int i = 0; i < c.count; ++i) {
    const DevStage& s = c.st[i];
    if (s.mul != 1 || s.s1 != 0 || s.add != 0 || s.lo > s.hi) return false;
    out->stage[i] = cvmhip_stage{CVMHIP_STAGE_CLAMP_SHIFT, 0, s.s2, s.lo, s.hi};
  }
  return true;
}

}  // namespace

extern "C" {

int cvmhip_fold_requant(const int32_t* bias, int oc, int64_t max_abs_acc, const cvmhip_chain* chain,
                        const cvmhip_chain* chain2, int has_residual, int32_t* bias_out, cvmhip_chain* chain_out,
                        cvmhip_chain* chain2_out) {
  if (oc < 1 || max_abs_acc < 0 || !bias_out || !chain_out || !chain2_out) return 0;
  DevChain c1, c2;
  if (!make_chain(chain, &c1) || !make_chain(has_residual ? chain2 : nullptr, &c2)) return 0;
  int64_t total = 0;   // what goes into the bias
  if (c1.count >= 1) {
    if (!plain_stage(c1.st[0])) return 0;
    total = c1.st[0].add;
    // the rounding term of the stage behind the residual add passes through chain1's only shift
    if (has_residual && c1.count == 1 && c2.count >= 1 && plain_stage(c2.st[0]) && c2.st[0].add != 0) {
      const int64_t t2 = c2.st[0].add;
      const int64_t through = t2 * ((int64_t)1 << c1.st[0].s2);
      if (through > (1ll << 30) || through < -(1ll << 30)) return 0;
      total += through;
      c2.st[0].lo = sat_add(c2.st[0].lo, t2);
      c2.st[0].hi = sat_add(c2.st[0].hi, t2);
      c2.st[0].add = 0;
    }
    c1.st[0].lo = sat_add(c1.st[0].lo, total);
    c1.st[0].hi = sat_add(c1.st[0].hi, total);
    c1.st[0].add = 0;
  } else if (has_residual && c2.count >= 1 && plain_stage(c2.st[0]) && c2.st[0].add != 0) {
    // no stage in front of the residual add: chain2's rounding term goes straight into the bias
    total = c2.st[0].add;
    c2.st[0].lo = sat_add(c2.st[0].lo, total);
    c2.st[0].hi = sat_add(c2.st[0].hi, total);
    c2.st[0].add = 0;
  }
  if (total == 0) return 0;
  // acc + bias + total must not wrap for any channel
  const int64_t mag = total < 0 ? -total : total;
  for (int i = 0; i < oc; ++i) {
    const int64_t b = bias ? bias[i] : 0;
    if ((b < 0 ? -b : b) + max_abs_acc + mag > INT32_MAX) return 0;
  }
  if (!to_public(c1, chain_out) || !to_public(c2, chain2_out)) return 0;
  for (int i = 0; i < oc; ++i) bias_out[i] = (int32_t)((bias ? bias[i] : 0) + total);
  return 1;
}

int cvmhip_chain_apply_host(const cvmhip_chain* chain, const int32_t* in, int64_t n, int32_t* out) {
  DevChain c;
  if (!make_chain(chain, &c) || !in || !out || n < 0) return arg_error("chain_apply_host");
  for (int64_t i = 0; i < n; ++i) {
    int32_t v = in[i];
    for (int t = 0; t < c.count; ++t) {
      const DevStage& s = c.st[t];
      v = v < s.lo ? s.lo : (v > s.hi ? s.hi : v);
      if (s.mul != 1) v = (int32_t)((uint32_t)v * (uint32_t)s.mul);
      v = (int32_t)((uint32_t)(v >> s.s1) + (uint32_t)s.add) >> s.s2;
    }
    out[i] = v;
  }
  return CVMHIP_OK;
}

}  // extern "C"
