// NITI's integer cross-entropy gradient (ti_loss.py:5-36) as one launch: one wavefront per sample.
//
// The reference evaluates a base-2 soft-max of the int8 logits in float32 tensor operations, truncates to
// integers twice on the way and rounds the result to int8 with StoShift(.., 4).  Every float32 operation
// of that sequence is kept, in the same order and with the same intermediate types (int64 sums of truncated
// values, float32 products and quotients).  The one operation whose result differs between math libraries,
// 2 ** s, is evaluated by a fixed sequence of IEEE double operations (exp2_contract below) that a host can
// repeat bit for bit, so the whole gradient is reproducible across devices.
#include "common.h"
#include "requant_math.h"

namespace niti {
namespace {

struct LossArgs {
  const int8_t* out;       // [n][classes] logits
  const int32_t* out_exp;  // exponent of the logits (device scalar)
  const int64_t* target;   // [n]
  const int32_t* rand;     // [n][classes], low four bits used
  int8_t* grad;            // [n][classes]
  int n, classes, trunc;
};

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

__device__ inline long long wave_sum_i64(long long v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const int lo = __shfl_xor(static_cast<int>(v & 0xFFFFFFFFLL), off, 64);
    const int hi = __shfl_xor(static_cast<int>(v >> 32), off, 64);
    v += (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo);
  }
  return v;
}

// One wavefront per sample, lanes over the classes.  The per-class terms are functions of the logit alone, so
// recomputing them in each of the three passes gives the same bits as the reference's stored tensors.
__global__ __launch_bounds__(256) void loss_grad_kernel(const LossArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.n) return;
  const int8_t* v = a.out + static_cast<long long>(row) * a.classes;
  const int e = *a.out_exp;
  const bool big = e > -7;
  const bool up = e >= 0;
  const float p2 = exp2f(static_cast<float>(up ? e : -e));   // exact power of two
  float off = 0.0f;
  // small exponents (ti_loss.py:26-30): 2^(1-2e) + v 2^(1-e) + v^2 in 64-bit integers that wrap like the tensor's
  const int sh2 = 1 - 2 * e, sh1 = 1 - e;
  const unsigned long long c2 = (!big && sh2 < 64) ? 1ULL << sh2 : 0ULL;
  auto small_term = [&](int x) {
    const unsigned long long lin = sh1 < 64 ? static_cast<unsigned long long>(static_cast<long long>(x)) << sh1 : 0ULL;
    return static_cast<long long>(c2 + lin + static_cast<unsigned long long>(static_cast<long long>(x) * x));
  };
  if (big) {
    float m = -INFINITY;
    for (int j = lane; j < a.classes; j += 64) m = fmaxf(m, scaled_logit(v[j], p2, up));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    off = m - 10.0f;
  }
  auto numer = [&](int j) -> float {   // out_grad before the normalisation, as float32
    if (!big) return static_cast<float>(small_term(v[j]));
    const float s = fmaxf(scaled_logit(v[j], p2, up) - off, 0.0f);
    return exp2_contract(s) - 1.0f;
  };
  long long sum = 0;   // out_grad.sum(1, dtype=int64): truncation of every term (ti_loss.py:31)
  for (int j = lane; j < a.classes; j += 64) sum += big ? static_cast<long long>(numer(j)) : small_term(v[j]);
  const float fsum = static_cast<float>(wave_sum_i64(sum));
  long long tsum = 0;  // ti_loss.py:34: int64 sum of the truncated normalised values
  for (int j = lane; j < a.classes; j += 64) tsum += static_cast<long long>(numer(j) * 2048.0f / fsum);
  tsum = wave_sum_i64(tsum);
  const long long t = a.target[row];
  const bool trunc = a.trunc != 0;
  for (int j = lane; j < a.classes; j += 64) {
    float g = numer(j) * 2048.0f / fsum;
    if (j == t) g = g - static_cast<float>(tsum);
    const int x = static_cast<int>(g);   // .type(torch.int32)
    const long long idx = static_cast<long long>(row) * a.classes + j;
    a.grad[idx] = static_cast<int8_t>(round_one<NITI_ROUND_STOCHASTIC>(x, 4, trunc, a.rand[idx] & 15));
  }
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" int niti_loss_grad_i8(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, const int32_t* rand,
                                 int8_t* grad, int n, int classes, int div_mode, void* stream) {
  clear_error();
  if (out_val == nullptr || out_exp == nullptr || target == nullptr || rand == nullptr || grad == nullptr)
    return fail(NITI_ERR_INVALID_ARG, "loss_grad: null pointer");
  if (n <= 0 || classes <= 0) return fail(NITI_ERR_INVALID_ARG, "loss_grad: n=%d classes=%d", n, classes);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "loss_grad: div_mode=%d", div_mode);
  const LossArgs a{out_val, out_exp, target, rand, grad, n, classes, div_mode == NITI_DIV_TRUNC ? 1 : 0};
  hipLaunchKernelGGL(loss_grad_kernel, dim3((n + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("loss_grad");
}
