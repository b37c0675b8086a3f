// Re-layout helpers around the convolution kernel: fills, the flipped/transposed filter the
// data gradient consumes, the outer<->inner byte transposition the weight gradient and the
// transposed GEMM forms consume, and the int32 post pass of split-k results.
#include "common.h"

namespace niti {
namespace {

__global__ void fill_u32_kernel(uint32_t* dst, int64_t n, uint32_t value) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = value;
}

// dst[c][r][s][k] = w[k][R-1-r][S-1-s][c]; one thread per destination byte (k fastest)
__global__ void filter_flip_transpose_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ dst, int K, int R,
                                             int S, int C) {
  const int64_t total = static_cast<int64_t>(K) * R * S * C;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int k = static_cast<int>(i % K);
    int64_t t = i / K;
    const int s = static_cast<int>(t % S);
    t /= S;
    const int r = static_cast<int>(t % R);
    const int c = static_cast<int>(t / R);
    dst[i] = w[((static_cast<int64_t>(k) * R + (R - 1 - r)) * S + (S - 1 - s)) * C + c];
  }
}

// src [A][B][C] -> dst [C][B][Apad] (bytes).  Grid: (ceil(Apad/64), ceil(C/64), B); the block
// moves a 64(a) x 64(c) byte tile through LDS so both the reads (along c) and the writes
// (along a) are contiguous 64-byte rows.
__global__ __launch_bounds__(256) void transpose_outer_inner_i8_kernel(const int8_t* __restrict__ src,
                                                                        int8_t* __restrict__ dst, int A, int B, int C,
                                                                        int Apad) {
  __shared__ int8_t tile[64][64 + 4];
  const int a0 = blockIdx.x * 64, c0 = blockIdx.y * 64, b = blockIdx.z;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int aa = a0 + i, cc = c0 + tx;
    int8_t v = 0;
    if (aa < A && cc < C) v = src[(static_cast<int64_t>(aa) * B + b) * C + cc];
    tile[i][tx] = v;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int cc = c0 + i, aa = a0 + tx;
    if (cc < C && aa < Apad) dst[(static_cast<int64_t>(cc) * B + b) * Apad + aa] = tile[tx][i];
  }
}

__global__ void post_i32_kernel(int32_t* v, int64_t n, int roundtrip, uint32_t* absmax) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  uint32_t lmax = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    int t = v[i];
    if (roundtrip) {
      t = f32_roundtrip(t);
      v[i] = t;
    }
    const uint32_t u = uabs(t);
    lmax = u > lmax ? u : lmax;
  }
  if (absmax != nullptr) fold_absmax(absmax, lmax);
}

inline int grid_for(int64_t n, int block, int cap = 8192) {
  int64_t g = (n + block - 1) / block;
  if (g < 1) g = 1;
  return static_cast<int>(g > cap ? cap : g);
}

}  // namespace

int launch_fill_u32(uint32_t* dst, int64_t n, uint32_t value, hipStream_t stream) {
  if (n <= 0) return NITI_OK;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n, 256)), dim3(256), 0, stream, dst, n, value);
  return check_launch("fill_u32");
}

int launch_filter_flip_transpose(const int8_t* w, int8_t* dst, int K, int R, int S, int C, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(K) * R * S * C;
  hipLaunchKernelGGL(filter_flip_transpose_kernel, dim3(grid_for(total, 256)), dim3(256), 0, stream, w, dst, K, R, S, C);
  return check_launch("filter_flip_transpose");
}

int launch_transpose_outer_inner_i8(const int8_t* src, int8_t* dst, int A, int B, int C, int Apad,
                                    hipStream_t stream) {
  if (B > 65535) return fail(NITI_ERR_UNSUPPORTED, "transpose: middle extent %d > 65535", B);
  dim3 grid((Apad + 63) / 64, (C + 63) / 64, B);
  if (grid.y > 65535u) return fail(NITI_ERR_UNSUPPORTED, "transpose: inner extent %d too large", C);
  hipLaunchKernelGGL(transpose_outer_inner_i8_kernel, grid, dim3(256), 0, stream, src, dst, A, B, C, Apad);
  return check_launch("transpose_outer_inner_i8");
}

int launch_post_i32(int32_t* v, int64_t n, bool roundtrip, uint32_t* absmax, hipStream_t stream) {
  if (n <= 0 || (!roundtrip && absmax == nullptr)) return NITI_OK;
  hipLaunchKernelGGL(post_i32_kernel, dim3(grid_for(n, 256, 2048)), dim3(256), 0, stream, v, n, roundtrip ? 1 : 0, absmax);
  return check_launch("post_i32");
}

}  // namespace niti
