// Arithmetic of the weighted sampler, shared bit for bit with the CPU oracle: every step is an
// exact integer conversion, an IEEE-754 division or an explicitly fused multiply-add, so both
// sides round identically.
#ifndef DGS_CSRC_WEIGHTS_H_
#define DGS_CSRC_WEIGHTS_H_

#include "common.h"

namespace dgs {

// -ln((x + 0.5) / 2^32): u = t / 2^33 with t = 2x + 1 = m * 2^e, m folded into
// (sqrt(1/2), sqrt(2)]; ln m = 2 atanh(s) with s = (m - 1) / (m + 1), series to s^21.
__device__ __forceinline__ double neg_log_u32(uint32_t x) {
#pragma clang fp contract(off)
  const uint64_t t = 2ull * x + 1ull;
  int e = 63 - __builtin_clzll(t);
  double m = double(t) * __longlong_as_double(int64_t(1023 - e) << 52);  // exact
  if (m > 0x1.6a09e667f3bcdp+0) {
    m *= 0.5;
    ++e;
  }
  const double f = m - 1.0;  // exact
  const double s = f / (2.0 + f);
  const double z = s * s;
  double p = 0x1.8618618618618p-5;             // 1/21
  p = __builtin_fma(p, z, 0x1.af286bca1af28p-5);  // 1/19
  p = __builtin_fma(p, z, 0x1.e1e1e1e1e1e1ep-5);  // 1/17
  p = __builtin_fma(p, z, 0x1.1111111111111p-4);  // 1/15
  p = __builtin_fma(p, z, 0x1.3b13b13b13b14p-4);  // 1/13
  p = __builtin_fma(p, z, 0x1.745d1745d1746p-4);  // 1/11
  p = __builtin_fma(p, z, 0x1.c71c71c71c71cp-4);  // 1/9
  p = __builtin_fma(p, z, 0x1.2492492492492p-3);  // 1/7
  p = __builtin_fma(p, z, 0x1.999999999999ap-3);  // 1/5
  p = __builtin_fma(p, z, 0x1.5555555555555p-2);  // 1/3
  p = __builtin_fma(p, z, 1.0);
  const double r = s * p;
  return __builtin_fma(double(33 - e), 0x1.62e42fefa39efp-1, -2.0 * r);
}

// Race key of neighbour position p: a unit exponential variate (from the position's Philox word
// x) over the weight, as the bits of a non-negative double (they order like the values).  A
// weight that is not > 0 gets +inf with p in the low bits, so such keys are distinct and order by
// position.  Position p of a row owns word p & 3 of the row's Philox block with counter word
// 0x80000000 | (p >> 2).
__device__ __forceinline__ uint64_t race_key(uint32_t x, float weight, uint32_t p) {
#pragma clang fp contract(off)
  const double w = double(weight);
  if (!(w > 0.0)) return 0x7ff0000000000000ull | p;
  return uint64_t(__double_as_longlong(neg_log_u32(x) / w));
}

// Scale of a row's integer shares: 32 - E with 2^(E-1) <= row_max < 2^E; row_max finite and > 0.
__device__ __forceinline__ int quantum_shift(float row_max) {
  const uint64_t bits = uint64_t(__double_as_longlong(double(row_max)));  // normal as a double
  return 32 - (int((bits >> 52) & 0x7ff) - 1022);
}

// Integer share of a weight in its row: floor(w * 2^shift) < 2^32, exact because the scale is a
// power of two; sums of shares are exact in any order, which is what lets a parallel scan and a
// sequential one agree.  0 for weights that are not > 0.
__device__ __forceinline__ uint64_t weight_quantum(float weight, int shift) {
  if (!(weight > 0.0f)) return 0;
  return uint64_t(__double2uint_rz(ldexp(double(weight), shift)));
}

// What a row's shares are measured against: `shift` when the largest weight is finite and > 0.
struct QuantumScale {
  int shift;
  bool none;      // no weight > 0: the row has no shares at all
  bool infinite;  // the largest weight is +inf: infinite weights share 1, finite ones 0
};
__device__ __forceinline__ QuantumScale quantum_scale(float row_max) {
  QuantumScale s;
  s.none = !(row_max > 0.0f);
  s.infinite = row_max > 3.4028234663852886e38f;
  s.shift = (s.none || s.infinite) ? 0 : quantum_shift(row_max);
  return s;
}
__device__ __forceinline__ uint64_t weight_quantum(float weight, const QuantumScale& s) {
  if (s.none) return 0;
  if (s.infinite) return weight > 3.4028234663852886e38f ? 1 : 0;
  return weight_quantum(weight, s.shift);
}

// Draw j of `row` (block 0x40000000 | j) reduced to [0, n): multiply-shift with rejection on the
// block's first 64 bits, the second 64 bits accepted unconditionally.
__device__ __forceinline__ uint64_t philox_bounded64(uint64_t seed, uint32_t stream, int64_t row, uint32_t j,
                                                     uint64_t n) {
  const PhiloxWords b = philox4x32_10(0x40000000u | j, stream, uint32_t(uint64_t(row)),
                                      uint32_t(uint64_t(row) >> 32), uint32_t(seed), uint32_t(seed >> 32));
  uint64_t x = uint64_t(b.w[0]) | (uint64_t(b.w[1]) << 32);
  const uint64_t lo = x * n;
  if (lo < n && lo < (0ull - n) % n) x = uint64_t(b.w[2]) | (uint64_t(b.w[3]) << 32);
  return __umul64hi(x, n);
}

}  // namespace dgs
#endif
