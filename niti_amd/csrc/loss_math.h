// Scalar pieces of NITI's integer cross-entropy gradient (ti_loss.py:5-36) shared by the kernels that evaluate it.
#pragma once
#include "common.h"

namespace niti {

// no fused multiply-add: the reference runs every operation as a kernel of its own
#pragma clang fp contract(off)

// ti_loss.py:10-24 for one logit: 2^max(s - offset, 0) - 1 with s = v * 47274 / 2^15 * 2^e
__device__ inline float scaled_logit(int v, float p2, bool up) {
  const float s = static_cast<float>(static_cast<long long>(v) * 47274) / 32768.0f;
  return up ? s * p2 : s / p2;
}

// 2^s for s >= 0: n = floor(s), x = (s - n) ln2, Horner's rule over 1/k! (k = 18 .. 0) in doubles with one rounded
// product and one rounded sum per step (no fused multiply-add), result = float(p 2^n).  Truncation error < 2^-60, so
// this is the correctly rounded float32 power except within ~2^-52 (relative) of a rounding boundary.
__device__ inline float exp2_contract(float s) {
  constexpr double c[19] = {
      0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,  0x1.5555555555555p-3,  0x1.5555555555555p-5,
      0x1.1111111111111p-7,  0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13, 0x1.a01a01a01a01ap-16, 0x1.71de3a556c734p-19,
      0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26, 0x1.1eed8eff8d898p-29, 0x1.6124613a86d09p-33, 0x1.93974a8c07c9dp-37,
      0x1.ae7f3e733b81fp-41, 0x1.ae7f3e733b81fp-45, 0x1.952c77030ad4ap-49, 0x1.6827863b97d97p-53};
  const double d = static_cast<double>(s);
  const double n = floor(d);
  const double x = (d - n) * 0x1.62e42fefa39efp-1;   // contraction is off for this file (pragma above)
  double p = c[18];
#pragma unroll
  for (int k = 17; k >= 0; --k) {
    p = p * x;
    p = p + c[k];
  }
  return static_cast<float>(ldexp(p, static_cast<int>(n)));
}

// ti_loss.py:26-30 for one logit x with exponent e <= -7: 2^(1-2e) + x 2^(1-e) + x^2 in 64-bit integers that wrap
// like the tensor's
__device__ inline long long loss_small_term(int x, int e) {
  const int sh2 = 1 - 2 * e, sh1 = 1 - e;
  const unsigned long long c2 = sh2 < 64 ? 1ULL << sh2 : 0ULL;
  const unsigned long long lin = sh1 < 64 ? static_cast<unsigned long long>(static_cast<long long>(x)) << sh1 : 0ULL;
  return static_cast<long long>(c2 + lin + static_cast<unsigned long long>(static_cast<long long>(x) * x));
}

}  // namespace niti
