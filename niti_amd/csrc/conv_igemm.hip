// int8 implicit-GEMM convolution forward on the gfx950 matrix cores.
//
// GEMM view: rows = output pixels m = (n,p,q), columns = output channels k, reduction over
// kg = (r,s,c).  NHWC activations and KRSC filters are both contiguous along the reduction
// index in 16-byte pieces (C % 16 == 0), so both operands stream from HBM with 16-byte
// coalesced loads into LDS tiles [128 rows][64 reduction bytes] and are consumed by
// v_mfma_i32_32x32x32_i8 (one 16-byte ds_read_b128 per lane per operand fragment).
//
// Workgroup: 256 threads = 4 wavefronts in a 2x2 arrangement, each owning a 64 pixel x 64
// channel patch of the 128x128 output tile = 2x2 MFMA tiles = 64 accumulator VGPRs.  The
// filter fragment is the MFMA "A" operand and the pixel fragment the "B" operand, which
// leaves every lane holding 4 consecutive output channels of one pixel per register quad:
// the int32 result goes out as 16-byte stores.  LDS rows are padded to 80 bytes so that the
// 16 lanes served together by a ds_read_b128 hit 16 distinct bank groups.
#include <stdlib.h>

#include "common.h"
#include "conv_args.h"

namespace niti {
namespace {

constexpr int BM = 128;  // pixels per workgroup
constexpr int BN = 128;  // output channels per workgroup
constexpr int BK = 64;   // reduction bytes per main-loop step
constexpr int LD = 80;   // padded LDS row pitch in bytes

template <bool kSplitK>
__global__ __launch_bounds__(256, 2) void conv_igemm_i8_kernel(const ConvArgs a) {
  __shared__ __attribute__((aligned(16))) int8_t smem[2][2][BM * LD];  // [stage][0: pixels, 1: filters]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m0 = blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  const int kit_begin = kSplitK ? static_cast<int>(blockIdx.z) * a.kiters_per_split : 0;
  const int kit_end = kSplitK ? min(kit_begin + a.kiters_per_split, a.kiters) : a.kiters;

  // ---- global -> LDS staging: thread owns 16-byte piece `chunk` of rows lrow and lrow+64
  const int chunk = tid & 3;
  const int lrow = tid >> 2;
  int hb[2], wb[2];
  long long xbase[2];
  bool mvalid[2], nvalid[2];
  const int8_t* wrow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = m0 + lrow + 64 * i;
    mvalid[i] = m < a.M;
    const int mm = mvalid[i] ? m : 0;
    const int n = mm / (a.P * a.Q);
    const int pq = mm - n * a.P * a.Q;
    const int p = pq / a.Q;
    const int q = pq - p * a.Q;
    hb[i] = p * a.stride - a.pad;
    wb[i] = q * a.stride - a.pad;
    xbase[i] = static_cast<long long>(n) * a.H * a.W * a.C;
    const int ko = n0 + lrow + 64 * i;
    nvalid[i] = ko < a.K;
    wrow[i] = a.w + static_cast<long long>(nvalid[i] ? ko : 0) * a.Kg;
  }
  int kg = kit_begin * BK + chunk * 16;
  int r, s, c;
  {
    const int rs = kg / a.C;
    c = kg - rs * a.C;
    r = rs / a.S;
    s = rs - r * a.S;
  }

  v4i ra[2], rb[2];
  auto gload = [&]() {
    const bool kvalid = kg < a.Kg;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int h = hb[i] + r;
      const int ww = wb[i] + s;
      const bool ok = mvalid[i] && kvalid && static_cast<unsigned>(h) < static_cast<unsigned>(a.H) &&
                      static_cast<unsigned>(ww) < static_cast<unsigned>(a.W);
      v4i va = {0, 0, 0, 0};
      if (ok) va = *reinterpret_cast<const v4i*>(a.x + xbase[i] + (static_cast<long long>(h) * a.W + ww) * a.C + c);
      ra[i] = va;
      v4i vb = {0, 0, 0, 0};
      if (nvalid[i] && kvalid) vb = *reinterpret_cast<const v4i*>(wrow[i] + kg);
      rb[i] = vb;
    }
  };
  auto advance = [&]() {
    kg += BK;
    c += BK;
    while (c >= a.C) {
      c -= a.C;
      if (++s == a.S) {
        s = 0;
        ++r;
      }
    }
  };
  auto sstore = [&](int st) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<v4i*>(&smem[st][0][(lrow + 64 * i) * LD + chunk * 16]) = ra[i];
      *reinterpret_cast<v4i*>(&smem[st][1][(lrow + 64 * i) * LD + chunk * 16]) = rb[i];
    }
  };

  // ---- MFMA main loop
  const int wm = wave & 1;   // which 64-pixel half
  const int wn = wave >> 1;  // which 64-channel half
  const int lr = lane & 31;
  const int lk = lane >> 5;
  v16i acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  if (kit_begin < kit_end) {
    gload();
    advance();
    sstore(0);
  }
  __syncthreads();
  for (int it = kit_begin; it < kit_end; ++it) {
    const int st = (it - kit_begin) & 1;
    const bool more = it + 1 < kit_end;
    if (more) {
      gload();
      advance();
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      v4i wf[2], pf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        wf[i] = *reinterpret_cast<const v4i*>(&smem[st][1][(wn * 64 + i * 32 + lr) * LD + kk * 32 + lk * 16]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        pf[j] = *reinterpret_cast<const v4i*>(&smem[st][0][(wm * 64 + j * 32 + lr) * LD + kk * 32 + lk * 16]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], pf[j], acc[i][j], 0, 0, 0);
    }
    if (more) sstore(st ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  acc[i][j][4g+e] = channel n0+wn*64+i*32+8g+4*lk+e of pixel m0+wm*64+j*32+lr
  const bool roundtrip = !kSplitK && (a.flags & NITI_EPI_F32_ROUNDTRIP);
  uint32_t lmax = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int m = m0 + wm * 64 + j * 32 + lr;
    long long obase = 0;
    if (m < a.M && !a.dense_out) {
      const int n = m / (a.P * a.Q);
      const int pq = m - n * a.P * a.Q;
      const int p = pq / a.Q;
      const int q = pq - p * a.Q;
      obase = n * a.ysN + p * a.ysP + q * a.ysQ;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int ch = n0 + wn * 64 + i * 32 + g * 8 + lk * 4;
        v4i v;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int t = acc[i][j][4 * g + e];
          if (roundtrip) t = f32_roundtrip(t);
          v[e] = t;
          const uint32_t u = uabs(t);
          lmax = u > lmax ? u : lmax;
        }
        if (m >= a.M) continue;
        if (!kSplitK && a.dense_out && ch + 3 < a.K) {
          *reinterpret_cast<v4i*>(a.y + static_cast<long long>(m) * a.K + ch) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (ch + e >= a.K) continue;
            const long long idx = a.dense_out ? static_cast<long long>(m) * a.K + ch + e : obase + (ch + e) * a.ysK;
            if (kSplitK) atomicAdd(a.y + idx, v[e]);
            else a.y[idx] = v[e];
          }
        }
      }
    }
  }
  if (!kSplitK && a.absmax != nullptr) fold_absmax(a.absmax, lmax);
}

}  // namespace

static int tile_override_from_env() {
  static const int tile = [] {   // read once (initialisation of a function-local static is thread-safe)
    const char* e = getenv("NITI_CONV_TILE");
    const int v = e != nullptr ? atoi(e) : 0;
    return (v < 0 || v > 6) ? 0 : v;
  }();
  return tile;
}

int launch_conv_igemm(const ConvProblem& p, hipStream_t stream) {
  ConvArgs a;
  a.x = p.x; a.w = p.w; a.y = p.y; a.absmax = p.absmax;
  a.N = p.N; a.H = p.H; a.W = p.W; a.C = p.C; a.K = p.K; a.R = p.R; a.S = p.S;
  a.stride = p.stride; a.pad = p.pad;
  a.P = (p.H + 2 * p.pad - p.R) / p.stride + 1;
  a.Q = (p.W + 2 * p.pad - p.S) / p.stride + 1;
  if (a.P <= 0 || a.Q <= 0) return fail(NITI_ERR_INVALID_ARG, "conv: empty output (%d x %d)", a.P, a.Q);
  const long long M = static_cast<long long>(p.N) * a.P * a.Q;
  const long long Kg = static_cast<long long>(p.R) * p.S * p.C;
  if (M > 0x7fffffffLL - BM || Kg > 0x7fffffffLL - 2 * BK)
    return fail(NITI_ERR_UNSUPPORTED, "conv: N*P*Q=%lld or R*S*C=%lld exceeds 2^31", M, Kg);
  if (p.C % 16 != 0) return fail(NITI_ERR_UNSUPPORTED, "conv: C=%d must be a multiple of 16", p.C);
  a.M = static_cast<int>(M);
  a.Kg = static_cast<int>(Kg);
  a.kiters = (a.Kg + BK - 1) / BK;
  a.ysN = p.ysN; a.ysP = p.ysP; a.ysQ = p.ysQ; a.ysK = p.ysK;
  a.dense_out = (p.ysK == 1 && p.ysQ == p.K && p.ysP == static_cast<long long>(a.Q) * p.K &&
                 p.ysN == static_cast<long long>(a.P) * a.Q * p.K && p.K % 4 == 0) ? 1 : 0;
  a.flags = p.flags;
  a.x_bytes = static_cast<long long>(p.N) * p.H * p.W * p.C;
  a.w_bytes = static_cast<long long>(p.K) * a.Kg;
  a.tile_override = tile_override_from_env();
  a.y_bytes = a.dense_out ? static_cast<long long>(a.M) * p.K * 4 : 0;
  a.pq_shift = a.q_shift = -1;
  {
    const int pq = a.P * a.Q;
    if ((pq & (pq - 1)) == 0 && (a.Q & (a.Q - 1)) == 0) {
      a.pq_shift = __builtin_ctz(pq);
      a.q_shift = __builtin_ctz(a.Q);
    }
  }
  int split = p.split_k < 1 ? 1 : p.split_k;
  if (split > a.kiters) split = a.kiters;
  a.kiters_per_split = (a.kiters + split - 1) / split;
  split = (a.kiters + a.kiters_per_split - 1) / a.kiters_per_split;
  if (conv_mfma_supported(a)) return launch_conv_mfma(a, split, stream);
  dim3 grid((a.M + BM - 1) / BM, (p.K + BN - 1) / BN, split);
  if (grid.y > 65535u || grid.z > 65535u) return fail(NITI_ERR_UNSUPPORTED, "conv: K=%d too large", p.K);
  if (split > 1)
    hipLaunchKernelGGL(conv_igemm_i8_kernel<true>, grid, dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL(conv_igemm_i8_kernel<false>, grid, dim3(256), 0, stream, a);
  return check_launch("conv_igemm_i8");
}

}  // namespace niti
