// Per-element shift-round-clip of the integer requantisation, shared by the stand-alone requantisation
// kernels and the convolution kernel that requantises its own sums.
#pragma once
#include "common.h"

namespace niti {

__device__ inline int clip127(long long v) { return static_cast<int>(v > 127 ? 127 : (v < -127 ? -127 : v)); }

// quotient and magnitude of the remainder of x / 2^s: floor division or truncation
__device__ inline void split_pow2(long long x, int s, bool trunc, long long& q, long long& rem) {
  if (!trunc || x >= 0) {
    q = x >> s;
    rem = x - (q << s);
  } else {
    const long long m = -x;
    q = -(m >> s);
    rem = m & ((1LL << s) - 1);
  }
}

// s >= 1.  u: random integer in [0, 2^s) for NITI_ROUND_STOCHASTIC, ignored otherwise
template <int kMethod>
__device__ inline int round_one(int x, int s, bool trunc, int u) {
  if (kMethod == NITI_ROUND_NEAREST) {
    const long long half = 1LL << (s - 1);
    if (!trunc) return clip127((static_cast<long long>(x) + half) >> s);
    const long long m = x < 0 ? -static_cast<long long>(x) : static_cast<long long>(x);
    const long long q = (m + half) >> s;
    return clip127(x < 0 ? -q : q);
  }
  long long q, rem;
  split_pow2(x, s, trunc, q, rem);
  const int sg = (x > 0) - (x < 0);
  if (kMethod == NITI_ROUND_STOCHASTIC) return clip127(q + (rem > static_cast<long long>(u) ? sg : 0));
  const int h = s >> 1;
  const long long hi = rem >> h;
  long long lo = rem & ((1LL << h) - 1);
  if (s & 1) lo <<= 1;
  return clip127(q + (hi > lo ? sg : 0));
}

// The same results as round_one for the methods that need no random input, in 32-bit arithmetic
// (1 <= s <= 31): floor((x + 2^(s-1)) / 2^s) = (x >> s) + bit s-1 of x, and remainders are masks.
template <int kMethod>
__host__ __device__ inline int round_one32(int x, int s, bool trunc) {
  static_assert(kMethod == NITI_ROUND_NEAREST || kMethod == NITI_ROUND_PSEUDO_STOCHASTIC, "no random input here");
  const bool neg = x < 0;
  const uint32_t m = neg ? 0u - static_cast<uint32_t>(x) : static_cast<uint32_t>(x);
  const bool by_magnitude = trunc && neg;
  int q;
  uint32_t rem;
  if (by_magnitude) {
    q = -static_cast<int>(m >> s);
    rem = m & ((1u << s) - 1u);
  } else {
    q = x >> s;
    rem = static_cast<uint32_t>(x) & ((1u << s) - 1u);
  }
  int r;
  if (kMethod == NITI_ROUND_NEAREST) {
    const int up = static_cast<int>((rem >> (s - 1)) & 1u);
    r = by_magnitude ? q - up : q + up;
  } else {
    const int h = s >> 1;
    const uint32_t hi = rem >> h;
    uint32_t lo = rem & ((1u << h) - 1u);
    if (s & 1) lo <<= 1;
    const int sg = (x > 0) - (x < 0);
    r = q + (hi > lo ? sg : 0);
  }
  return r > 127 ? 127 : (r < -127 ? -127 : r);
}

// StoShift in 32-bit arithmetic (1 <= s <= 31): one step away from zero when the magnitude of the remainder exceeds
// the low s bits of the random integer u (ti_torch.py:33-46: prob <= rand_num -> 0, else sign(input)).
__host__ __device__ inline int round_sto32(int x, int s, bool trunc, int u) {
  const bool neg = x < 0;
  const uint32_t m = neg ? 0u - static_cast<uint32_t>(x) : static_cast<uint32_t>(x);
  const uint32_t mask = (1u << s) - 1u;
  int q;
  uint32_t rem;
  if (trunc && neg) {
    q = -static_cast<int>(m >> s);
    rem = m & mask;
  } else {
    q = x >> s;
    rem = static_cast<uint32_t>(x) & mask;
  }
  const int sg = (x > 0) - (x < 0);
  const int r = q + (rem > (static_cast<uint32_t>(u) & mask) ? sg : 0);
  return r > 127 ? 127 : (r < -127 ? -127 : r);
}

// Four rounded values -> four bytes (value e in byte e), two's complement low bytes.
__device__ inline uint32_t pack4_i8(int r0, int r1, int r2, int r3) {
  // v_perm_b32: selector byte 0x00-0x03 picks a byte of the second operand, 0x04-0x07 of the first, 0x0c is zero
  const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(r1), static_cast<uint32_t>(r0), 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(r3), static_cast<uint32_t>(r2), 0x0c0c0400u);
  return lo | (hi << 16);
}

// Nearest rounding with floor division for 1 <= s and |x| < 2^(s + 7) (true when s comes from the tensor's own
// range): floor((x + 2^(s-1)) / 2^s) = ((x >> (s-1)) + 1) >> 1, then clip to [lo, 127] (lo = -127, or 0 for a
// fused ReLU).  Three shifts/adds and one median instead of the general path's dozen operations.
__device__ inline int round_nearest_floor_fast(int x, int sm1, int lo) {
  const int r = ((x >> sm1) + 1) >> 1;
  return min(max(r, lo), 127);
}

// The same for four values at once, as the dword of their four int8 results: after the first shift the values fit
// 16 bits (|x| < 2^(s + 7) gives |x >> (s-1)| <= 256; the conversion saturates beyond), so the increment, the second
// shift and the clip run on packed 16-bit pairs - 15 instructions for four values instead of 23.  Exact whenever
// |x >> (s-1)| < 32767; the callers' shift is never smaller than what their own largest magnitude needs (a predicted
// shift only ever raises it), so |x >> (s-1)| <= 256 for every value they pass.
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ inline uint32_t round4_nearest_floor_fast(int x0, int x1, int x2, int x3, int sm1, int lo) {
  v2s a = __builtin_amdgcn_cvt_pk_i16(x0 >> sm1, x1 >> sm1);
  v2s b = __builtin_amdgcn_cvt_pk_i16(x2 >> sm1, x3 >> sm1);
  const v2s one = {1, 1}, lo2 = {static_cast<short>(lo), static_cast<short>(lo)}, hi2 = {127, 127};
  a = (a + one) >> 1;
  b = (b + one) >> 1;
  a = __builtin_elementwise_min(__builtin_elementwise_max(a, lo2), hi2);
  b = __builtin_elementwise_min(__builtin_elementwise_max(b, lo2), hi2);
  // bytes 0 and 2 of each pair
  return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b), __builtin_bit_cast(uint32_t, a), 0x06040200u);
}

// 0xFF in every byte of m that is positive as an int8, 0x00 elsewhere (the ReLU-backward test on four activations)
__host__ __device__ inline uint32_t positive_bytes(uint32_t m) {
  const uint32_t nz = (((m & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | m) & 0x80808080u;  // bit 7 where the byte is non-zero
  const uint32_t pos = nz & ~m;                                               // ... and its sign bit is clear
  return (pos >> 7) * 0xFFu;
}

// 0xFF in every byte where a and b agree
__host__ __device__ inline uint32_t equal_bytes(uint32_t a, uint32_t b) {
  const uint32_t z = a ^ b;
  const uint32_t nz = (((z & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | z) & 0x80808080u;   // bit 7 of the bytes that differ
  return ((nz ^ 0x80808080u) >> 7) * 0xFFu;
}

// the larger of four signed bytes, byte by byte: each byte in the high half of a 16-bit lane keeps its order there
__device__ inline uint32_t max_i8x4(uint32_t a, uint32_t b) {
  typedef short s2_t __attribute__((ext_vector_type(2)));
  union U { uint32_t u; s2_t s; };
  U ah, bh, al, bl, mh, ml;
  ah.u = a & 0xFF00FF00u;
  bh.u = b & 0xFF00FF00u;
  al.u = (a << 8) & 0xFF00FF00u;
  bl.u = (b << 8) & 0xFF00FF00u;
  mh.s = __builtin_elementwise_max(ah.s, bh.s);
  ml.s = __builtin_elementwise_max(al.s, bl.s);
  return mh.u | (ml.u >> 8);
}

// shift < 1: the reference converts int32 to int8 by keeping the low byte
__device__ inline int wrap_to_i8(int x) { return static_cast<int>(static_cast<int8_t>(static_cast<uint32_t>(x) & 0xFFu)); }

}  // namespace niti
