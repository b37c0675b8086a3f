// NHWC int8 max pooling forward / backward (bandwidth kernels) and the grouped int8
// convolution with float output that stands in for the reference's cuDNN group_conv.
// Pooling threads own 16 consecutive channels of one pixel (one 16-byte load/store) when
// C % 16 == 0, one channel otherwise.
#include "common.h"
#include "requant_math.h"

namespace niti {
namespace {

template <int V>
struct Bytes;
template <>
struct Bytes<16> {
  v4i v;
  __device__ void load(const int8_t* p) { v = *reinterpret_cast<const v4i*>(p); }
  __device__ void store(int8_t* p) const { *reinterpret_cast<v4i*>(p) = v; }
  __device__ int get(int i) const { return static_cast<int8_t>((static_cast<uint32_t>(v[i >> 2]) >> (8 * (i & 3))) & 0xFFu); }
};
template <>
struct Bytes<1> {
  int8_t v;
  __device__ void load(const int8_t* p) { v = *p; }
  __device__ void store(int8_t* p) const { *p = v; }
  __device__ int get(int) const { return v; }
};

template <int V>
__device__ inline void pack_store(int8_t* p, const int* vals) {
  if (V == 16) {
    v4i o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t w = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) w |= (static_cast<uint32_t>(vals[4 * d + e]) & 0xFFu) << (8 * e);
      o[d] = static_cast<int>(w);
    }
    *reinterpret_cast<v4i*>(p) = o;
  } else {
    *p = static_cast<int8_t>(vals[0]);
  }
}

struct PoolArgs {
  const int8_t* x;
  const int8_t* y;
  const int8_t* dy;
  int8_t* out;
  int N, H, W, C, P, Q, ks, stride, pad, ties_all;
  int relu;   // backward: also zero the positions whose input is not positive (a ReLU in front of the pooling)
};

template <int V>
__global__ __launch_bounds__(256) void maxpool_fwd_kernel(const PoolArgs a) {
  const int CV = a.C / V;
  const int64_t total = static_cast<int64_t>(a.N) * a.P * a.Q * CV;
  const int64_t gstride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += gstride) {
    const int cv = static_cast<int>(i % CV);
    int64_t t = i / CV;
    const int q = static_cast<int>(t % a.Q);
    t /= a.Q;
    const int p = static_cast<int>(t % a.P);
    const int n = static_cast<int>(t / a.P);
    int best[V];
#pragma unroll
    for (int e = 0; e < V; ++e) best[e] = -128;
    for (int kh = 0; kh < a.ks; ++kh) {
      const int h = p * a.stride - a.pad + kh;
      if (h < 0 || h >= a.H) continue;
      for (int kw = 0; kw < a.ks; ++kw) {
        const int w = q * a.stride - a.pad + kw;
        if (w < 0 || w >= a.W) continue;
        Bytes<V> b;
        b.load(a.x + ((static_cast<int64_t>(n) * a.H + h) * a.W + w) * a.C + cv * V);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const int v = b.get(e);
          best[e] = v > best[e] ? v : best[e];
        }
      }
    }
    pack_store<V>(a.out + i * V, best);
  }
}

// One thread per input position: visit every window that covers it and add dy when this
// position is the window's (first / any) maximum.
template <int V>
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const PoolArgs a) {
  const int CV = a.C / V;
  const int64_t total = static_cast<int64_t>(a.N) * a.H * a.W * CV;
  const int64_t gstride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += gstride) {
    const int cv = static_cast<int>(i % CV);
    int64_t t = i / CV;
    const int w = static_cast<int>(t % a.W);
    t /= a.W;
    const int h = static_cast<int>(t % a.H);
    const int n = static_cast<int>(t / a.H);
    Bytes<V> xs;
    xs.load(a.x + i * V);
    int acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0;
    // windows p with p*stride - pad <= h <= p*stride - pad + ks - 1
    int plo = h + a.pad - a.ks + 1;
    plo = plo <= 0 ? 0 : (plo + a.stride - 1) / a.stride;
    int phi = (h + a.pad) / a.stride;
    phi = phi >= a.P ? a.P - 1 : phi;
    int qlo = w + a.pad - a.ks + 1;
    qlo = qlo <= 0 ? 0 : (qlo + a.stride - 1) / a.stride;
    int qhi = (w + a.pad) / a.stride;
    qhi = qhi >= a.Q ? a.Q - 1 : qhi;
    for (int p = plo; p <= phi; ++p) {
      for (int q = qlo; q <= qhi; ++q) {
        const int64_t o = ((static_cast<int64_t>(n) * a.P + p) * a.Q + q) * a.C + cv * V;
        Bytes<V> ys, ds;
        ys.load(a.y + o);
        ds.load(a.dy + o);
        bool hit[V];
#pragma unroll
        for (int e = 0; e < V; ++e) hit[e] = xs.get(e) == ys.get(e);
        if (!a.ties_all) {
          // an earlier position (scan order kh, kw) holding the maximum takes the gradient instead
          const int mykh = h - (p * a.stride - a.pad), mykw = w - (q * a.stride - a.pad);
          for (int kh = 0; kh <= mykh; ++kh) {
            const int hh = p * a.stride - a.pad + kh;
            if (hh < 0 || hh >= a.H) continue;
            const int kwend = kh == mykh ? mykw : a.ks;
            for (int kw = 0; kw < kwend; ++kw) {
              const int ww = q * a.stride - a.pad + kw;
              if (ww < 0 || ww >= a.W) continue;
              Bytes<V> o2;
              o2.load(a.x + ((static_cast<int64_t>(n) * a.H + hh) * a.W + ww) * a.C + cv * V);
#pragma unroll
              for (int e = 0; e < V; ++e) hit[e] = hit[e] && (o2.get(e) != ys.get(e));
            }
          }
        }
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += hit[e] ? ds.get(e) : 0;
      }
    }
    if (a.relu) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = xs.get(e) > 0 ? acc[e] : 0;
    }
    pack_store<V>(a.out + i * V, acc);
  }
}

// The layers' case: 2 x 2 windows, stride 2, no padding, even H and W, C % 16 == 0.  Windows do not overlap, so a
// lane owns one window x 16 channels: six 16-byte loads, byte-parallel compares, four 16-byte stores.
template <bool kAll>
__global__ __launch_bounds__(256) void maxpool2x2_bwd_kernel(const PoolArgs a) {
  const int CV = a.C >> 4;
  const int64_t total = static_cast<int64_t>(a.N) * a.P * a.Q * CV;
  const int64_t gstride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t rowb = static_cast<int64_t>(a.W) * a.C;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += gstride) {
    const uint32_t pix = static_cast<uint32_t>(i / CV);           // (n * P + p) * Q + q < 2^31 (checked on the host)
    const uint32_t cv = static_cast<uint32_t>(i - static_cast<int64_t>(pix) * CV);
    const uint32_t q = pix % static_cast<uint32_t>(a.Q);
    const uint32_t np = pix / static_cast<uint32_t>(a.Q);         // n * P + p; input row 2 * np since H = 2 P
    const int64_t x0 = (static_cast<int64_t>(np) * 2 * a.W + 2 * q) * a.C + cv * 16;
    const v4i y = *reinterpret_cast<const v4i*>(a.y + i * 16);
    const v4i d = *reinterpret_cast<const v4i*>(a.dy + i * 16);
    v4i x[4];
    x[0] = *reinterpret_cast<const v4i*>(a.x + x0);
    x[1] = *reinterpret_cast<const v4i*>(a.x + x0 + a.C);
    x[2] = *reinterpret_cast<const v4i*>(a.x + x0 + rowb);
    x[3] = *reinterpret_cast<const v4i*>(a.x + x0 + rowb + a.C);
    v4i o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint32_t taken = 0;   // bytes whose gradient an earlier position of the window (scan order) already received
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t eq = equal_bytes(static_cast<uint32_t>(x[k][e]), static_cast<uint32_t>(y[e]));
        uint32_t keep = kAll ? eq : eq & ~taken;
        if (a.relu) keep &= positive_bytes(static_cast<uint32_t>(x[k][e]));
        o[k][e] = static_cast<int>(static_cast<uint32_t>(d[e]) & keep);
        taken |= eq;
      }
    }
    *reinterpret_cast<v4i*>(a.out + x0) = o[0];
    *reinterpret_cast<v4i*>(a.out + x0 + a.C) = o[1];
    *reinterpret_cast<v4i*>(a.out + x0 + rowb) = o[2];
    *reinterpret_cast<v4i*>(a.out + x0 + rowb + a.C) = o[3];
  }
}

struct GroupConvArgs {
  const int8_t* x;
  const int8_t* w;
  float* y;
  int N, H, W, C, K, R, S, Cg, P, Q, stride, pad, dil, kper;
};

// One wavefront per output element; lanes stride over the (r,s,cg) reduction so filter reads
// are contiguous, then a wavefront sum.
__global__ __launch_bounds__(256) void group_conv_i8_f32_kernel(const GroupConvArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = (static_cast<int64_t>(gridDim.x) * blockDim.x) >> 6;
  const int64_t total = static_cast<int64_t>(a.N) * a.P * a.Q * a.K;
  const int red = a.R * a.S * a.Cg;
  for (int64_t o = wave; o < total; o += nwaves) {
    const int k = static_cast<int>(o % a.K);
    int64_t t = o / a.K;
    const int q = static_cast<int>(t % a.Q);
    t /= a.Q;
    const int p = static_cast<int>(t % a.P);
    const int n = static_cast<int>(t / a.P);
    const int g = k / a.kper;
    int sum = 0;
    for (int j = lane; j < red; j += 64) {
      const int cg = j % a.Cg;
      const int rs = j / a.Cg;
      const int s = rs % a.S, r = rs / a.S;
      const int h = p * a.stride - a.pad + r * a.dil;
      const int ww = q * a.stride - a.pad + s * a.dil;
      if (h < 0 || h >= a.H || ww < 0 || ww >= a.W) continue;
      const int xv = a.x[((static_cast<int64_t>(n) * a.H + h) * a.W + ww) * a.C + g * a.Cg + cg];
      const int wv = a.w[static_cast<int64_t>(k) * red + j];
      sum += xv * wv;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) a.y[o] = static_cast<float>(sum);
  }
}

inline int grid_for(int64_t n, int block, int cap = 8192) {
  int64_t g = (n + block - 1) / block;
  if (g < 1) g = 1;
  return static_cast<int>(g > cap ? cap : g);
}

int check_pool(const char* who, int N, int H, int W, int C, int ks, int stride, int pad, int* P, int* Q) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0) return fail(NITI_ERR_INVALID_ARG, "%s: non-positive extent", who);
  if (ks <= 0 || stride <= 0 || pad < 0 || 2 * pad > ks)
    return fail(NITI_ERR_INVALID_ARG, "%s: kernel %d stride %d pad %d", who, ks, stride, pad);
  *P = (H + 2 * pad - ks) / stride + 1;
  *Q = (W + 2 * pad - ks) / stride + 1;
  if (H + 2 * pad < ks || W + 2 * pad < ks) return fail(NITI_ERR_INVALID_ARG, "%s: window larger than input", who);
  return NITI_OK;
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" int niti_maxpool_i8_fwd(const int8_t* x, int8_t* y, int N, int H, int W, int C, int ks, int stride, int pad,
                                   void* stream) {
  clear_error();
  int P, Q;
  int st = check_pool("maxpool_fwd", N, H, W, C, ks, stride, pad, &P, &Q);
  if (st != NITI_OK) return st;
  if (x == nullptr || y == nullptr) return fail(NITI_ERR_INVALID_ARG, "maxpool_fwd: null pointer");
  PoolArgs a{x, nullptr, nullptr, y, N, H, W, C, P, Q, ks, stride, pad, 0, 0};
  const bool vec = C % 16 == 0 && aligned16(x) && aligned16(y);
  const int64_t total = static_cast<int64_t>(N) * P * Q * (vec ? C / 16 : C);
  if (vec) hipLaunchKernelGGL(maxpool_fwd_kernel<16>, dim3(grid_for(total, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  else hipLaunchKernelGGL(maxpool_fwd_kernel<1>, dim3(grid_for(total, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("maxpool_fwd");
}

extern "C" int niti_maxpool_i8_bwd(const int8_t* y, const int8_t* dy, const int8_t* x, int8_t* dx, int N, int H, int W,
                                   int C, int ks, int stride, int pad, int ties, void* stream) {
  clear_error();
  int P, Q;
  int st = check_pool("maxpool_bwd", N, H, W, C, ks, stride, pad, &P, &Q);
  if (st != NITI_OK) return st;
  if (x == nullptr || y == nullptr || dy == nullptr || dx == nullptr) return fail(NITI_ERR_INVALID_ARG, "maxpool_bwd: null pointer");
  const int relu = (ties & NITI_POOL_BWD_RELU) != 0;
  ties &= ~NITI_POOL_BWD_RELU;
  if (ties != NITI_TIES_FIRST && ties != NITI_TIES_ALL) return fail(NITI_ERR_INVALID_ARG, "maxpool_bwd: ties=%d", ties);
  PoolArgs a{x, y, dy, dx, N, H, W, C, P, Q, ks, stride, pad, ties == NITI_TIES_ALL, relu};
  const bool vec = C % 16 == 0 && aligned16(x) && aligned16(y) && aligned16(dy) && aligned16(dx);
  if (vec && ks == 2 && stride == 2 && pad == 0 && H % 2 == 0 && W % 2 == 0 && static_cast<int64_t>(N) * P * Q < 0x7fffffffLL) {
    const int64_t windows = static_cast<int64_t>(N) * P * Q * (C / 16);
    const dim3 grid(grid_for(windows, 256, 1 << 20));
    if (ties == NITI_TIES_ALL) hipLaunchKernelGGL(maxpool2x2_bwd_kernel<true>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
    else hipLaunchKernelGGL(maxpool2x2_bwd_kernel<false>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a);
    return check_launch("maxpool2x2_bwd");
  }
  const int64_t total = static_cast<int64_t>(N) * H * W * (vec ? C / 16 : C);
  if (vec) hipLaunchKernelGGL(maxpool_bwd_kernel<16>, dim3(grid_for(total, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  else hipLaunchKernelGGL(maxpool_bwd_kernel<1>, dim3(grid_for(total, 256)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("maxpool_bwd");
}

extern "C" int niti_group_conv_i8_f32(const int8_t* x, const int8_t* w, float* y, int N, int H, int W, int C, int K,
                                      int R, int S, int Cg, int stride, int pad, int dilation, int groups,
                                      void* stream) {
  clear_error();
  if (x == nullptr || w == nullptr || y == nullptr) return fail(NITI_ERR_INVALID_ARG, "group_conv: null pointer");
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || Cg <= 0 || groups <= 0 || stride <= 0 ||
      dilation <= 0 || pad < 0)
    return fail(NITI_ERR_INVALID_ARG, "group_conv: non-positive extent");
  if (C != groups * Cg || K % groups != 0)
    return fail(NITI_ERR_INVALID_ARG, "group_conv: C=%d, K=%d do not match groups=%d x Cg=%d", C, K, groups, Cg);
  const int P = (H + 2 * pad - dilation * (R - 1) - 1) / stride + 1;
  const int Q = (W + 2 * pad - dilation * (S - 1) - 1) / stride + 1;
  if (P <= 0 || Q <= 0) return fail(NITI_ERR_INVALID_ARG, "group_conv: empty output");
  GroupConvArgs a{x, w, y, N, H, W, C, K, R, S, Cg, P, Q, stride, pad, dilation, K / groups};
  const int64_t total = static_cast<int64_t>(N) * P * Q * K;
  hipLaunchKernelGGL(group_conv_i8_f32_kernel, dim3(grid_for(total * 64, 256, 16384)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), a);
  return check_launch("group_conv_i8_f32");
}
