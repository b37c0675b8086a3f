// Integer requantisation kernels: per-tensor max |x|, shift-round-clip back to int8 (nearest,
// stochastic with supplied random integers, pseudo-stochastic), the fused gradient rounding +
// weight update, ReLU forward/backward.  All are single-pass HBM-bandwidth kernels that move
// 16 int32 (64 bytes in, 16 bytes out) per thread per step; the shift is derived on the
// device from the max the producer kernel left in memory.
#include "common.h"
#include "requant_math.h"

namespace niti {
namespace {

__global__ __launch_bounds__(256) void absmax_i32_kernel(const int32_t* __restrict__ x, int64_t n, uint32_t* absmax) {
  const int64_t nv = n >> 2;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  uint32_t lmax = 0;
  const v4i* xv = reinterpret_cast<const v4i*>(x);
  for (int64_t i = t0; i < nv; i += stride) {
    const v4i v = xv[i];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t u = uabs(v[e]);
      lmax = u > lmax ? u : lmax;
    }
  }
  for (int64_t i = (nv << 2) + t0; i < n; i += stride) {
    const uint32_t u = uabs(x[i]);
    lmax = u > lmax ? u : lmax;
  }
  fold_absmax(absmax, lmax);
}

struct RequantArgs {
  const int32_t* x;
  int8_t* y;        // requant: output.  grad update: optional rounded gradient
  int8_t* w;        // grad update only
  const int32_t* rand;
  const uint32_t* absmax;
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
  int64_t n;
  int target_bits, trunc, bw_mode;
  unsigned flags;
};

// kUpdate == false: y = requant(x).  kUpdate == true: g = requant(x); w = clip(w - g); y (optional) = g
template <int kMethod, bool kUpdate>
__global__ __launch_bounds__(256) void requant_kernel(const RequantArgs a) {
  const int shift = bitwidth_of(*a.absmax, a.bw_mode) - a.target_bits;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const int sh = shift > 0 ? shift : 0;
    if (a.shift_out != nullptr) *a.shift_out = sh;
    if (a.exp_out != nullptr)
      *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
  }
  // random integers are reduced to their low `shift` bits: values already in [0, 2^shift) pass
  // unchanged, wider uniform bits become uniform in [0, 2^shift) without the host knowing shift
  const int rm = shift >= 1 ? static_cast<int>((1u << (shift > 31 ? 31 : shift)) - 1u) : 0;
  const v4i rmask = {rm, rm, rm, rm};
  const bool trunc = a.trunc != 0;
  const bool relu = (a.flags & NITI_RQ_RELU) != 0;
  auto one = [&](int x, int u) -> int {
    int r;
    if (shift >= 1) r = round_one<kMethod>(x, shift, trunc, u);
    else r = wrap_to_i8(x);
    if (relu && r < 0) r = 0;
    return r;
  };
  const int64_t nv = a.n >> 4;  // groups of 16 elements
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const v4i* xv = reinterpret_cast<const v4i*>(a.x);
  const v4i* uv = reinterpret_cast<const v4i*>(a.rand);
  for (int64_t i = t0; i < nv; i += stride) {
    v4i out;
    v4i wv = {0, 0, 0, 0};
    if (kUpdate) wv = reinterpret_cast<const v4i*>(a.w)[i];
    v4i neww;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const v4i v = xv[i * 4 + d];
      v4i u = {0, 0, 0, 0};
      if (kMethod == NITI_ROUND_STOCHASTIC && shift >= 1) u = uv[i * 4 + d] & rmask;
      uint32_t packed = 0, packedw = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = one(v[e], u[e]);
        packed |= (static_cast<uint32_t>(r) & 0xFFu) << (8 * e);
        if (kUpdate) {
          const int wold = static_cast<int>(static_cast<int8_t>((static_cast<uint32_t>(wv[d]) >> (8 * e)) & 0xFFu));
          packedw |= (static_cast<uint32_t>(clip127(wold - r)) & 0xFFu) << (8 * e);
        }
      }
      out[d] = static_cast<int>(packed);
      neww[d] = static_cast<int>(packedw);
    }
    if (kUpdate) {
      reinterpret_cast<v4i*>(a.w)[i] = neww;
      if (a.y != nullptr) reinterpret_cast<v4i*>(a.y)[i] = out;
    } else {
      reinterpret_cast<v4i*>(a.y)[i] = out;
    }
  }
  for (int64_t i = (nv << 4) + t0; i < a.n; i += stride) {
    int u = 0;
    if (kMethod == NITI_ROUND_STOCHASTIC && shift >= 1) u = a.rand[i] & rmask[0];
    const int r = one(a.x[i], u);
    if (kUpdate) {
      a.w[i] = static_cast<int8_t>(clip127(static_cast<int>(a.w[i]) - r));
      if (a.y != nullptr) a.y[i] = static_cast<int8_t>(r);
    } else {
      a.y[i] = static_cast<int8_t>(r);
    }
  }
}

__global__ __launch_bounds__(256) void weight_update_kernel(int8_t* w, const int8_t* __restrict__ g, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    w[i] = static_cast<int8_t>(clip127(static_cast<int>(w[i]) - static_cast<int>(g[i])));
}

// ---- input quantiser (TiFloatToInt8, ti_torch.py:341-356) with the layout change that follows it (ti_net.py:19) ----
// r = max |x| over the batch (float bits of non-negative values order like unsigned integers)
__global__ __launch_bounds__(256) void absmax_f32_kernel(const float* __restrict__ x, int64_t n, uint32_t* __restrict__ out) {
  __shared__ uint32_t wmax[4];
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  uint32_t m = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint32_t b = __float_as_uint(x[i]) & 0x7FFFFFFFu;
    m = b > m ? b : m;
  }
  m = wave_max_u32(m);
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x < 64) fold_absmax(out, threadIdx.x < 4 ? wmax[threadIdx.x] : 0u);
}

// bw = ceil(log2 r); y = int8(clamp(round_half_even(x * 2^(bits - bw)), -128, 127)), float NCHW -> int8 NHWC with the
// channels zero-padded to cpad; exp_out = bw - bits.  The product and the rounding are the reference's float32 operations.
__global__ __launch_bounds__(256) void quantize_f32_i8_kernel(const float* __restrict__ x, int8_t* __restrict__ y, int64_t pixels,
                                                              int C, int HW, int cpad, const uint32_t* __restrict__ absmax_bits,
                                                              int32_t* exp_out, int bits) {
  const float r = __uint_as_float(*absmax_bits);
  // ceil(log2 r) from the exponent and mantissa of r = m 2^e, 0.5 <= m < 1 (exact; a library log2f rounds k + log2(1 + d)
  // back to k for the first float32 values above 2^k, k >= 4, and differs between platforms there)
  int fe = 0;
  const float fm = frexpf(r, &fe);
  const int bw = fm == 0.5f ? fe - 1 : fe;
  const float scale = ldexpf(1.0f, bits - bw);
  if (blockIdx.x == 0 && threadIdx.x == 0 && exp_out != nullptr) *exp_out = r > 0.0f ? bw - bits : 0;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < pixels; p += stride) {
    const int64_t n = p / HW, hw = p - n * HW;
    const float* src = x + n * C * HW + hw;
    int8_t* dst = y + p * cpad;
    for (int c0 = 0; c0 < cpad; c0 += 4) {
      uint32_t word = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int c = c0 + e;
        int q = 0;
        if (c < C && r > 0.0f) {
          const float v = fminf(fmaxf(rintf(src[static_cast<int64_t>(c) * HW] * scale), -128.0f), 127.0f);
          q = static_cast<int>(v);
        }
        word |= (static_cast<uint32_t>(q) & 0xFFu) << (8 * e);
      }
      *reinterpret_cast<uint32_t*>(dst + c0) = word;
    }
  }
}

// y[m][f] = x[m][f] * mask[f] with mask bytes 0 / 1 (a keep / drop decision per feature); optionally exp_out = exp_in + add
__global__ __launch_bounds__(256) void mask_features_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ mask,
                                                            int8_t* __restrict__ y, int64_t rows, int features,
                                                            const int32_t* exp_in, int32_t* exp_out, int exp_add) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t0 == 0 && exp_out != nullptr) *exp_out = (exp_in != nullptr ? *exp_in : 0) + exp_add;
  const int fv = features >> 4;   // features % 16 == 0 (host check)
  const int64_t nv = rows * fv;
  for (int64_t i = t0; i < nv; i += stride) {
    const int f = static_cast<int>(i % fv);
    const v4i xv = reinterpret_cast<const v4i*>(x)[i];
    const v4i mv = reinterpret_cast<const v4i*>(mask)[f];
    v4i o;
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = xv[d] & static_cast<int>((static_cast<uint32_t>(mv[d]) & 0x01010101u) * 0xFFu);
    reinterpret_cast<v4i*>(y)[i] = o;
  }
}

// kBwd == false: y = max(x, 0).  kBwd == true: y = x(act) > 0 ? dy : 0
template <bool kBwd>
__global__ __launch_bounds__(256) void relu_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ dy,
                                                   int8_t* __restrict__ y, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const bool vec = aligned16_dev(x) && aligned16_dev(y) && (!kBwd || aligned16_dev(dy));
  const int64_t nv = vec ? (n >> 4) : 0;
  for (int64_t i = t0; i < nv; i += stride) {
    const v4i xv = reinterpret_cast<const v4i*>(x)[i];
    v4i dv = {0, 0, 0, 0};
    if (kBwd) dv = reinterpret_cast<const v4i*>(dy)[i];
    v4i o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t p = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int xe = static_cast<int8_t>((static_cast<uint32_t>(xv[d]) >> (8 * e)) & 0xFFu);
        const uint32_t src = kBwd ? ((static_cast<uint32_t>(dv[d]) >> (8 * e)) & 0xFFu) : (static_cast<uint32_t>(xe) & 0xFFu);
        p |= (xe > 0 ? src : 0u) << (8 * e);
      }
      o[d] = static_cast<int>(p);
    }
    reinterpret_cast<v4i*>(y)[i] = o;
  }
  for (int64_t i = (nv << 4) + t0; i < n; i += stride) y[i] = x[i] > 0 ? (kBwd ? dy[i] : x[i]) : static_cast<int8_t>(0);
}

inline int grid_for(int64_t work_items, int block, int cap = 4096) {
  int64_t g = (work_items + block - 1) / block;
  if (g < 1) g = 1;
  return static_cast<int>(g > cap ? cap : g);
}

template <bool kUpdate>
int launch_requant(const RequantArgs& a, int method, hipStream_t stream) {
  const dim3 grid(grid_for((a.n + 15) / 16, 256)), block(256);
  switch (method) {
    case NITI_ROUND_NEAREST:
      hipLaunchKernelGGL((requant_kernel<NITI_ROUND_NEAREST, kUpdate>), grid, block, 0, stream, a);
      break;
    case NITI_ROUND_STOCHASTIC:
      hipLaunchKernelGGL((requant_kernel<NITI_ROUND_STOCHASTIC, kUpdate>), grid, block, 0, stream, a);
      break;
    case NITI_ROUND_PSEUDO_STOCHASTIC:
      hipLaunchKernelGGL((requant_kernel<NITI_ROUND_PSEUDO_STOCHASTIC, kUpdate>), grid, block, 0, stream, a);
      break;
    default:
      return fail(NITI_ERR_INVALID_ARG, "requant: unknown rounding method %d", method);
  }
  return check_launch("requant");
}

int check_requant_common(const char* who, const void* x, int64_t n, const uint32_t* absmax, int target_bits, int method,
                         int div_mode, int bw_mode, const int32_t* rand) {
  if (n < 0) return fail(NITI_ERR_INVALID_ARG, "%s: n=%lld", who, static_cast<long long>(n));
  if (n == 0) return NITI_OK;
  if (x == nullptr || absmax == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (!aligned16(x)) return fail(NITI_ERR_INVALID_ARG, "%s: input must be 16-byte aligned", who);
  if (target_bits < 1 || target_bits > 7) return fail(NITI_ERR_INVALID_ARG, "%s: target_bits=%d outside 1..7", who, target_bits);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "%s: div_mode=%d", who, div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "%s: bw_mode=%d", who, bw_mode);
  if (method == NITI_ROUND_STOCHASTIC && (rand == nullptr || !aligned16(rand)))
    return fail(NITI_ERR_INVALID_ARG, "%s: stochastic rounding needs a 16-byte aligned rand tensor", who);
  return NITI_OK;
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" int niti_absmax_i32(const int32_t* x, int64_t n, uint32_t* absmax, void* stream) {
  clear_error();
  if (n < 0) return fail(NITI_ERR_INVALID_ARG, "absmax: n=%lld", static_cast<long long>(n));
  if (n == 0) return NITI_OK;
  if (x == nullptr || absmax == nullptr) return fail(NITI_ERR_INVALID_ARG, "absmax: null pointer");
  if (!aligned16(x)) return fail(NITI_ERR_INVALID_ARG, "absmax: input must be 16-byte aligned");
  hipLaunchKernelGGL(absmax_i32_kernel, dim3(grid_for((n + 3) / 4, 256, 2048)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), x, n, absmax);
  return check_launch("absmax_i32");
}

extern "C" int niti_requant_i32_i8(const int32_t* x, int8_t* y, int64_t n, const uint32_t* absmax, int target_bits,
                                   int method, int div_mode, int bw_mode, const int32_t* rand, unsigned flags,
                                   int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                   void* stream) {
  clear_error();
  int st = check_requant_common("requant", x, n, absmax, target_bits, method, div_mode, bw_mode, rand);
  if (st != NITI_OK || n == 0) return st;
  if (y == nullptr || !aligned16(y)) return fail(NITI_ERR_INVALID_ARG, "requant: output must be non-null and 16-byte aligned");
  RequantArgs a{x, y, nullptr, rand, absmax, shift_out, exp_a, exp_b, exp_out, n, target_bits, div_mode == NITI_DIV_TRUNC, bw_mode, flags};
  return launch_requant<false>(a, method, static_cast<hipStream_t>(stream));
}

extern "C" int niti_grad_update_i8(const int32_t* g, int8_t* w, int64_t n, const uint32_t* absmax, int mu, int method,
                                   int div_mode, int bw_mode, const int32_t* rand, int8_t* g8_out, int32_t* shift_out,
                                   const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream) {
  clear_error();
  int st = check_requant_common("grad_update", g, n, absmax, mu, method, div_mode, bw_mode, rand);
  if (st != NITI_OK || n == 0) return st;
  if (w == nullptr || !aligned16(w)) return fail(NITI_ERR_INVALID_ARG, "grad_update: weights must be non-null and 16-byte aligned");
  if (g8_out != nullptr && !aligned16(g8_out)) return fail(NITI_ERR_INVALID_ARG, "grad_update: g8_out must be 16-byte aligned");
  RequantArgs a{g, g8_out, w, rand, absmax, shift_out, exp_a, exp_b, exp_out, n, mu, div_mode == NITI_DIV_TRUNC, bw_mode, 0u};
  return launch_requant<true>(a, method, static_cast<hipStream_t>(stream));
}

extern "C" int niti_weight_update_i8(int8_t* w, const int8_t* g, int64_t n, void* stream) {
  clear_error();
  if (n < 0) return fail(NITI_ERR_INVALID_ARG, "weight_update: n=%lld", static_cast<long long>(n));
  if (n == 0) return NITI_OK;
  if (w == nullptr || g == nullptr) return fail(NITI_ERR_INVALID_ARG, "weight_update: null pointer");
  hipLaunchKernelGGL(weight_update_kernel, dim3(grid_for(n, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), w, g, n);
  return check_launch("weight_update");
}

extern "C" int niti_relu_i8_fwd(const int8_t* x, int8_t* y, int64_t n, void* stream) {
  clear_error();
  if (n < 0) return fail(NITI_ERR_INVALID_ARG, "relu: n=%lld", static_cast<long long>(n));
  if (n == 0) return NITI_OK;
  if (x == nullptr || y == nullptr) return fail(NITI_ERR_INVALID_ARG, "relu: null pointer");
  hipLaunchKernelGGL(relu_kernel<false>, dim3(grid_for((n + 15) / 16, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     x, static_cast<const int8_t*>(nullptr), y, n);
  return check_launch("relu_fwd");
}

extern "C" int niti_quantize_f32_i8(const float* x, int8_t* y, int N, int C, int H, int W, int cpad, int bits, uint32_t* absmax_bits,
                                    int32_t* exp_out, void* stream) {
  clear_error();
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || cpad < C || cpad % 4 != 0 || bits < 1 || bits > 7)
    return fail(NITI_ERR_INVALID_ARG, "quantize: N=%d C=%d H=%d W=%d cpad=%d bits=%d", N, C, H, W, cpad, bits);
  if (x == nullptr || y == nullptr || absmax_bits == nullptr) return fail(NITI_ERR_INVALID_ARG, "quantize: null pointer");
  if (reinterpret_cast<uintptr_t>(y) % 4 != 0) return fail(NITI_ERR_INVALID_ARG, "quantize: output must be 4-byte aligned");
  const int64_t pixels = static_cast<int64_t>(N) * H * W, n = pixels * C;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(absmax_f32_kernel, dim3(grid_for(n, 256, 1024)), dim3(256), 0, s, x, n, absmax_bits);
  hipLaunchKernelGGL(quantize_f32_i8_kernel, dim3(grid_for(pixels, 256)), dim3(256), 0, s, x, y, pixels, C, H * W, cpad, absmax_bits,
                     exp_out, bits);
  return check_launch("quantize");
}

extern "C" int niti_mask_features_i8(const int8_t* x, const int8_t* mask, int8_t* y, int64_t rows, int features,
                                     const int32_t* exp_in, int32_t* exp_out, int exp_add, void* stream) {
  clear_error();
  if (rows < 0 || features <= 0 || features % 16 != 0)
    return fail(NITI_ERR_INVALID_ARG, "mask_features: rows=%lld features=%d (a multiple of 16)", static_cast<long long>(rows), features);
  if (x == nullptr || mask == nullptr || y == nullptr) return fail(NITI_ERR_INVALID_ARG, "mask_features: null pointer");
  if (!aligned16(x) || !aligned16(mask) || !aligned16(y)) return fail(NITI_ERR_INVALID_ARG, "mask_features: pointers must be 16-byte aligned");
  const int64_t nv = rows * (features >> 4);
  hipLaunchKernelGGL(mask_features_kernel, dim3(grid_for(nv > 0 ? nv : 1, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), x, mask, y,
                     rows, features, exp_in, exp_out, exp_add);
  return check_launch("mask_features");
}

extern "C" int niti_relu_i8_bwd(const int8_t* act, const int8_t* dy, int8_t* dx, int64_t n, void* stream) {
  clear_error();
  if (n < 0) return fail(NITI_ERR_INVALID_ARG, "relu_bwd: n=%lld", static_cast<long long>(n));
  if (n == 0) return NITI_OK;
  if (act == nullptr || dy == nullptr || dx == nullptr) return fail(NITI_ERR_INVALID_ARG, "relu_bwd: null pointer");
  hipLaunchKernelGGL(relu_kernel<true>, dim3(grid_for((n + 15) / 16, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     act, dy, dx, n);
  return check_launch("relu_bwd");
}
