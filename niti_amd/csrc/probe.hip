// Measurement aid: a register-resident int8 MFMA loop (no LDS, no memory traffic inside the loop) over operands
// the caller supplies.  The rate this loop sustains is the matrix-unit ceiling for those operand VALUES: on MI355X
// the shader clock follows the power the multipliers draw, so uniform random int8 operands run at a markedly lower
// clock (and rate) than constant ones.  bench.py reports both next to the datasheet peak.
#include "common.h"

namespace niti {
namespace {

// 8 wavefronts per workgroup, each holding 2 x 2 accumulator tiles of 32 x 32 (the convolution kernel's register
// shape) and 2 + 6 operand fragments loaded once; `iters` rounds of 12 MFMAs.
__global__ __launch_bounds__(512, 2) void mfma_probe_kernel(const int8_t* __restrict__ operands, long long bytes, int iters,
                                                            int32_t* __restrict__ out, long long* __restrict__ clocks) {
  const int tid = threadIdx.x;
  v4i pc[2], wf[3][2];
  const long long frag = (static_cast<long long>(blockIdx.x) * 512 + tid) * 8;   // this lane's first 16-byte fragment
  const long long nfrag = bytes / 16;
  auto load = [&](int i) { return reinterpret_cast<const v4i*>(operands)[(frag + i) % nfrag]; };
  pc[0] = load(0);
  pc[1] = load(1);
#pragma unroll
  for (int s = 0; s < 3; ++s)
#pragma unroll
    for (int i = 0; i < 2; ++i) wf[s][i] = load(2 + s * 2 + i);
  v16i acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
  const long long c0 = __builtin_readcyclecounter();
  const long long w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[s][i], pc[j], acc[i][j], 0, 0, 0);
    // the accumulators wrap; keep the operands opaque so that the loop is not folded
#pragma unroll
    for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(pc[j]));
  }
  int sum = 0;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
  out[static_cast<long long>(blockIdx.x) * 512 + tid] = sum;
  if (blockIdx.x == 0 && tid == 0 && clocks != nullptr) {
    clocks[0] = __builtin_readcyclecounter() - c0;   // shader clocks
    clocks[1] = wall_clock64() - w0;                 // 100 MHz ticks
  }
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" int niti_mfma_probe_i8(const int8_t* operands, size_t operand_bytes, int workgroups, int iters, int32_t* out,
                                  int64_t* clocks, void* stream) {
  clear_error();
  if (operands == nullptr || out == nullptr || !aligned16(operands)) return fail(NITI_ERR_INVALID_ARG, "mfma_probe: null or misaligned pointer");
  if (operand_bytes < 128 || workgroups <= 0 || workgroups > 65535 || iters <= 0)
    return fail(NITI_ERR_INVALID_ARG, "mfma_probe: operand_bytes=%zu workgroups=%d iters=%d", operand_bytes, workgroups, iters);
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(workgroups), dim3(512), 0, static_cast<hipStream_t>(stream), operands,
                     static_cast<long long>(operand_bytes), iters, out, reinterpret_cast<long long*>(clocks));
  return check_launch("mfma_probe");
}
