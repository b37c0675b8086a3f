// Kernel argument block shared by the convolution kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace niti {

struct ConvArgs {
  const int8_t* x;   // [N,H,W,C]
  const int8_t* w;   // [K,R,S,C]
  int32_t* y;
  uint32_t* absmax;  // may be null
  int N, H, W, C, K, R, S, P, Q, stride, pad;
  int M, Kg;         // N*P*Q output pixels, R*S*C reduction bytes
  int kiters, kiters_per_split;
  long long ysN, ysP, ysQ, ysK;  // output strides in elements
  int dense_out;     // y is plain [M][K] with K % 4 == 0: 16-byte stores allowed
  unsigned flags;
  long long x_bytes, w_bytes;  // extents of x and w, for the buffer descriptors
  long long y_bytes;           // extent of a dense y (0 otherwise)
  int pq_shift, q_shift;       // log2(P*Q), log2(Q) when both are powers of two, else -1
  int tile_override;           // 0: heuristic; 1..4 force a tile configuration (tuning)
};

bool conv_mfma_supported(const ConvArgs& a);
int launch_conv_mfma(const ConvArgs& a, int split, hipStream_t stream);

}  // namespace niti
