// NITI's integer cross-entropy gradient (ti_loss.py:5-36) as one launch: one wavefront per sample.
//
// The reference evaluates a base-2 soft-max of the int8 logits in float32 tensor operations, truncates to
// integers twice on the way and rounds the result to int8 with StoShift(.., 4).  Every float32 operation
// of that sequence is kept, in the same order and with the same intermediate types (int64 sums of truncated
// values, float32 products and quotients).  The one operation whose result differs between math libraries,
// 2 ** s, is evaluated by a fixed sequence of IEEE double operations (exp2_contract below) that a host can
// repeat bit for bit, so the whole gradient is reproducible across devices.
#include "common.h"
#include "loss_math.h"
#include "requant_math.h"
#include "rng.h"

namespace niti {
namespace {

struct LossArgs {
  const int8_t* out;       // [n][classes] logits
  const int32_t* out_exp;  // exponent of the logits (device scalar)
  const int64_t* target;   // [n]
  const int32_t* rand;     // [n][classes], low four bits used; null: drawn from rng
  uint32_t* rng;           // generator state (rng.h), used when rand is null
  int8_t* grad;            // [n][classes]
  int n, classes, trunc;
};

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
  // Every wavefront reads the generator state, then the workgroup reports in: the last workgroup to do so starts the
  // next step, so no wavefront of this launch may still have its read ahead of it at that point.
  RngDraw draw{};
  if (a.rand == nullptr) draw = rng_read(a.rng);
  __syncthreads();
  if (a.rand == nullptr && threadIdx.x == 0) rng_arrive(a.rng, gridDim.x, draw);
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
    const int u = a.rand != nullptr ? a.rand[idx] & 15 : static_cast<int>(rng_word(draw, kRngStreamLoss, static_cast<uint32_t>(idx)) & 15u);
    a.grad[idx] = static_cast<int8_t>(round_one<NITI_ROUND_STOCHASTIC>(x, 4, trunc, u));
  }
}

}  // namespace
}  // namespace niti

using namespace niti;

static int loss_launch(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, const int32_t* rand, uint32_t* rng,
                       int8_t* grad, int n, int classes, int div_mode, void* stream) {
  clear_error();
  if (out_val == nullptr || out_exp == nullptr || target == nullptr || (rand == nullptr && rng == nullptr) || grad == nullptr)
    return fail(NITI_ERR_INVALID_ARG, "loss_grad: null pointer");
  if (n <= 0 || classes <= 0) return fail(NITI_ERR_INVALID_ARG, "loss_grad: n=%d classes=%d", n, classes);
  if (static_cast<long long>(n) * classes > 0x7FFFFFFFLL) return fail(NITI_ERR_UNSUPPORTED, "loss_grad: more than 2^31 logits");
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "loss_grad: div_mode=%d", div_mode);
  const LossArgs a{out_val, out_exp, target, rand, rng, grad, n, classes, div_mode == NITI_DIV_TRUNC ? 1 : 0};
  hipLaunchKernelGGL(loss_grad_kernel, dim3((n + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("loss_grad");
}

extern "C" int niti_loss_grad_i8(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, const int32_t* rand,
                                 int8_t* grad, int n, int classes, int div_mode, void* stream) {
  if (rand == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "loss_grad: null pointer");
  }
  return loss_launch(out_val, out_exp, target, rand, nullptr, grad, n, classes, div_mode, stream);
}

extern "C" int niti_loss_grad_i8_rng(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, uint32_t* rng,
                                     int8_t* grad, int n, int classes, int div_mode, void* stream) {
  if (rng == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "loss_grad: null pointer");
  }
  return loss_launch(out_val, out_exp, target, nullptr, rng, grad, n, classes, div_mode, stream);
}

// ---- the generator's words, for callers that want to see what a kernel will draw --------------------------------
namespace niti {
namespace {
__global__ __launch_bounds__(256) void rng_words_kernel(const uint32_t* state, uint32_t stream_id, uint32_t* out, long long n) {
  const RngDraw d = rng_read(state);
  const long long q = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;   // a lane writes four words
  if (4 * q >= n) return;
  uint32_t w[4];
  rng_words4(d, stream_id, static_cast<uint32_t>(q), w);
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (4 * q + i < n) out[4 * q + i] = w[i];
}
}  // namespace
}  // namespace niti

extern "C" int niti_rng_words_u32(const uint32_t* rng, uint32_t stream_id, uint32_t* out, size_t n, void* stream) {
  clear_error();
  if (rng == nullptr || (out == nullptr && n != 0)) return fail(NITI_ERR_INVALID_ARG, "rng_words: null pointer");
  if (n == 0) return NITI_OK;
  if (n > (1ULL << 34)) return fail(NITI_ERR_UNSUPPORTED, "rng_words: a stream has 2^34 words");
  const long long quads = static_cast<long long>((n + 3) / 4);
  hipLaunchKernelGGL(rng_words_kernel, dim3(static_cast<unsigned>((quads + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     rng, stream_id, out, static_cast<long long>(n));
  return check_launch("rng_words");
}
