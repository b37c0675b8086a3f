// Pipelined int8 implicit-GEMM convolution for gfx950: the fast path of launch_conv_igemm().
//
// Same GEMM view as conv_igemm.hip (rows = output pixels, columns = output channels,
// reduction over (r,s,c) in 64-byte steps) with three changes that matter on CDNA4:
//   * operand tiles go global -> LDS with buffer_load_dwordx4 ... lds (no VGPR staging, no
//     ds_write); padding pixels and out-of-range rows use an out-of-range buffer offset, for
//     which the hardware delivers zeros;
//   * a STAGES-deep ring of LDS tiles with one s_barrier per step; the wavefront waits on
//     vmcnt only for the stage it is about to consume, the younger stages stay in flight;
//   * LDS rows are 64 bytes, unpadded, with the 16-byte piece index XOR-swizzled by
//     (row >> 2) & 3, which makes the ds_read_b128 of the MFMA fragments conflict free.
// A workgroup is WVM x WVN wavefronts; each owns (WP*32 pixels) x (WC*32 channels) of the
// (WVM*WP*32) x (WVN*WC*32) output tile as WP x WC v_mfma_i32_32x32x32_i8 tiles.  The vector
// memory path delivers 64 bytes/clock/CU, so the tile must be large: loads per step are
// (BM+BN)*64 bytes for 2*BM*BN*64 ops.
#include "common.h"
#include "conv_args.h"

namespace niti {
namespace {

#define NITI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
constexpr int kOobOffset = -1;  // 0xFFFFFFFF: beyond any buffer, the load returns zeros

template <int N>
__device__ inline void wait_vmcnt() {
  // s_waitcnt vmcnt(N), leaving expcnt and lgkmcnt unconstrained (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | 0x0F70);
}

__device__ inline void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int WVM, int WVN, int WP, int WC, int STAGES, int BK, bool kSplitK>
__global__ __launch_bounds__(WVM * WVN * 64, (WVM * WVN == 8 ? 1 : 2)) void conv_mfma_kernel(const ConvArgs a) {
  constexpr int NW = WVM * WVN;
  constexpr int BM = WVM * WP * 32, BN = WVN * WC * 32;
  constexpr int STAGE_BYTES = (BM + BN) * BK;
  constexpr int PR = BK / 16;    // 16-byte pieces per LDS row
  constexpr int RPI = 64 / PR;   // rows filled by one load instruction
  constexpr int SWS = BK == 64 ? 2 : 1;  // swizzle: piece ^= (row >> SWS) & (PR - 1)
  constexpr int LA = BM / (RPI * NW), LB = BN / (RPI * NW);  // loads per thread per stage
  constexpr int NL = LA + LB;
  static_assert(BK == 64 || BK == 128, "reduction step is 64 or 128 bytes");
  static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "tile rows must split evenly over the wavefronts");
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m0 = blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  const int kit_begin = kSplitK ? static_cast<int>(blockIdx.z) * a.kiters_per_split : 0;
  const int kit_end = kSplitK ? min(kit_begin + a.kiters_per_split, a.kiters) : a.kiters;
  const int nk = kit_end - kit_begin;

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.w), 0, a.w_bytes, 0x00020000);

  // ---- loader state.  One load instruction fills RPI rows x BK bytes; lane -> (row lane/PR, piece lane%PR)
  const int rr = lane / PR;
  // the row index inside the tile is (wave + NW*i)*RPI + rr and NW*RPI is a multiple of 32, so the
  // swizzle bits come from wave*RPI + rr alone
  const int chunk = (lane % PR) ^ (((wave * RPI + rr) >> SWS) & (PR - 1));  // which 16 bytes of the row this lane fetches
  int pixoff[LA];
  unsigned tapmask[LA];
  int woff[LB];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    const int m = m0 + (wave + NW * i) * RPI + rr;
    unsigned mask = 0;
    int off = 0;
    if (m < a.M) {
      int n, p, q;
      if (a.pq_shift >= 0) {  // P*Q and Q are powers of two: shifts instead of divisions
        n = m >> a.pq_shift;
        const int pq = m & ((1 << a.pq_shift) - 1);
        p = pq >> a.q_shift;
        q = pq & ((1 << a.q_shift) - 1);
      } else {
        n = m / (a.P * a.Q);
        const int pq = m - n * a.P * a.Q;
        p = pq / a.Q;
        q = pq - p * a.Q;
      }
      const int hb = p * a.stride - a.pad, wb = q * a.stride - a.pad;
      off = ((n * a.H + hb) * a.W + wb) * a.C;
      // tap (r,s) is inside the image iff row r and column s are: build the R*S-bit mask from the two
      unsigned colmask = 0;
      for (int s = 0; s < a.S; ++s)
        if (static_cast<unsigned>(wb + s) < static_cast<unsigned>(a.W)) colmask |= 1u << s;
      for (int r = 0; r < a.R; ++r)
        if (static_cast<unsigned>(hb + r) < static_cast<unsigned>(a.H)) mask |= colmask << (r * a.S);
    }
    pixoff[i] = off;
    tapmask[i] = mask;
  }
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    const int ko = n0 + (wave + NW * i) * RPI + rr;
    woff[i] = ko < a.K ? ko * a.Kg : kOobOffset;   // rows past K: every load out of range
  }
  int kg = kit_begin * BK + chunk * 16;
  int tap, cc, delta;  // tap index r*S+s, channel offset, (r*W+s)*C+cc
  {
    tap = kg / a.C;
    cc = kg - tap * a.C;
    const int r = tap / a.S, s = tap - r * a.S;
    delta = (r * a.W + s) * a.C + cc;
  }
  int sidx = tap % a.S;  // s of the current tap, to step delta across filter rows

  auto issue = [&](int st) {
    int8_t* base = smem + st * STAGE_BYTES;
    const bool kvalid = kg < a.Kg;
    const unsigned tapbit = kvalid ? (1u << (tap & 31)) : 0u;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      const int off = (tapmask[i] & tapbit) ? pixoff[i] + delta : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, NITI_LDS(base + (wave + NW * i) * 1024), 16, off, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      const int off = (kvalid && woff[i] != kOobOffset) ? woff[i] + kg : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS(base + BM * BK + (wave + NW * i) * 1024), 16, off, 0, 0, 0);
    }
    // advance the reduction position by BK bytes
    kg += BK;
    cc += BK;
    delta += BK;
    while (cc >= a.C) {
      cc -= a.C;
      ++tap;                // next tap along s is the adjacent pixel: delta already points there
      if (++sidx == a.S) {  // wrapped to the next filter row: pixel (r+1, 0) instead of (r, S)
        sidx = 0;
        delta += (a.W - a.S) * a.C;
      }
    }
  };

  // ---- accumulators
  const int wm = wave % WVM, wn = wave / WVM;
  const int lr = lane & 31, lk = lane >> 5;
  const int swz = (lr >> SWS) & (PR - 1);
  v16i acc[WC][WP];
#pragma unroll
  for (int i = 0; i < WC; ++i)
#pragma unroll
    for (int j = 0; j < WP; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // ---- prologue: STAGES-1 stages in flight
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < nk) issue(s);

  for (int it = 0; it < nk; ++it) {
    // stage `it` is the oldest one in flight; younger ones (at most STAGES-2) may stay pending
    if (it + STAGES - 2 < nk) wait_vmcnt<(STAGES - 2) * NL>();
    else wait_vmcnt<0>();
    wg_barrier();
    if (it + STAGES - 1 < nk) issue((it + STAGES - 1) % STAGES);
    const int8_t* sa = smem + (it % STAGES) * STAGE_BYTES;  // pixels
    const int8_t* sb = sa + BM * BK;                         // filters
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      const int piece = ((2 * kk + lk) ^ swz) << 4;
      v4i wf[WC], pf[WP];
#pragma unroll
      for (int i = 0; i < WC; ++i)
        wf[i] = *reinterpret_cast<const v4i*>(sb + (wn * WC * 32 + i * 32 + lr) * BK + piece);
#pragma unroll
      for (int j = 0; j < WP; ++j)
        pf[j] = *reinterpret_cast<const v4i*>(sa + (wm * WP * 32 + j * 32 + lr) * BK + piece);
#pragma unroll
      for (int i = 0; i < WC; ++i)
#pragma unroll
        for (int j = 0; j < WP; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], pf[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue.  acc[i][j][4g+e] = channel n0+(wn*WC+i)*32+8g+4*lk+e of pixel m0+(wm*WP+j)*32+lr
  const bool roundtrip = !kSplitK && (a.flags & NITI_EPI_F32_ROUNDTRIP);
  uint32_t lmax = 0;
  if (!kSplitK && a.dense_out) {
    // Dense [M][K] int32 output: each wavefront turns its 32-pixel x (WC*32)-channel slabs around in
    // its own LDS patch so that a store instruction covers whole (WC*128)-byte runs of 4 pixel rows.
    constexpr int ROWB = WC * 32 * 4 + 16;  // padded row pitch of the patch, bytes
    static_assert(NW * 32 * ROWB <= STAGES * STAGE_BYTES, "epilogue patch must fit in the stage buffers");
    // range of this wavefront's accumulators: one max3 / min3 per two values
    int vmax = 0, vmin = 0;
#pragma unroll
    for (int i = 0; i < WC; ++i)
#pragma unroll
      for (int j = 0; j < WP; ++j)
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          vmax = max(vmax, max(acc[i][j][e], acc[i][j][e + 1]));
          vmin = min(vmin, min(acc[i][j][e], acc[i][j][e + 1]));
        }
    lmax = max(static_cast<uint32_t>(vmax), 0u - static_cast<uint32_t>(vmin));
    // the fp32 round trip is the identity up to 2^24: only a wavefront that holds a larger value pays for it
    const bool big = roundtrip && wave_max_u32(lmax) > (1u << 24);
    if (big) {
      lmax = 0;
#pragma unroll
      for (int i = 0; i < WC; ++i)
#pragma unroll
        for (int j = 0; j < WP; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int t = f32_roundtrip(acc[i][j][e]);
            acc[i][j][e] = t;
            const uint32_t u = uabs(t);
            lmax = u > lmax ? u : lmax;
          }
    }
    wg_barrier();  // every wavefront is done reading the stage buffers
    int8_t* patch = smem + wave * (32 * ROWB);
    constexpr int LPR = WC * 8;        // lanes per pixel row (16 bytes each)
    constexpr int RPS = 64 / LPR;      // pixel rows per store instruction
    const int rrow = lane / LPR, rcol = lane % LPR;
    const int ch = n0 + wn * WC * 32 + rcol * 4;
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
#pragma unroll
    for (int j = 0; j < WP; ++j) {
#pragma unroll
      for (int i = 0; i < WC; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const v4i v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          *reinterpret_cast<v4i*>(patch + lr * ROWB + (i * 32 + g * 8 + lk * 4) * 4) = v;
        }
      // same wavefront reads back what it wrote: LDS operations of one wavefront complete in order
      const int mrow = m0 + (wm * WP + j) * 32 + rrow;
#pragma unroll
      for (int t = 0; t < 32 / RPS; ++t) {
        const v4i v = *reinterpret_cast<const v4i*>(patch + (t * RPS + rrow) * ROWB + rcol * 16);
        const int m = mrow + t * RPS;
        // rows past M and channels past K go to an out-of-range offset, which the hardware drops
        const int off = (m < a.M && ch < a.K) ? (m * a.K + ch) * 4 : kOobOffset;
        __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < WP; ++j) {
      const int m = m0 + (wm * WP + j) * 32 + lr;
      long long obase = 0;
      if (m < a.M && !a.dense_out) {
        const int n = m / (a.P * a.Q);
        const int pq = m - n * a.P * a.Q;
        const int p = pq / a.Q;
        const int q = pq - p * a.Q;
        obase = n * a.ysN + p * a.ysP + q * a.ysQ;
      }
#pragma unroll
      for (int i = 0; i < WC; ++i) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int ch = n0 + (wn * WC + i) * 32 + g * 8 + lk * 4;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            int t = acc[i][j][4 * g + e];
            if (roundtrip) t = f32_roundtrip(t);
            const uint32_t u = uabs(t);
            lmax = u > lmax ? u : lmax;
            if (m >= a.M || ch + e >= a.K) continue;
            const long long idx = a.dense_out ? static_cast<long long>(m) * a.K + ch + e : obase + (ch + e) * a.ysK;
            if (kSplitK) atomicAdd(a.y + idx, t);
            else a.y[idx] = t;
          }
        }
      }
    }
  }
  if (!kSplitK && a.absmax != nullptr) fold_absmax(a.absmax, lmax);
}

template <int WVM, int WVN, int WP, int WC, int STAGES, int BK>
int launch_cfg(const ConvArgs& a_in, int split, hipStream_t stream) {
  constexpr int BM = WVM * WP * 32, BN = WVN * WC * 32;
  ConvArgs a = a_in;  // reduction steps counted in this configuration's BK
  a.kiters = (a.Kg + BK - 1) / BK;
  if (split > a.kiters) split = a.kiters;
  a.kiters_per_split = (a.kiters + split - 1) / split;
  split = (a.kiters + a.kiters_per_split - 1) / a.kiters_per_split;
  constexpr size_t lds = static_cast<size_t>(STAGES) * (BM + BN) * BK;
  dim3 grid((a.M + BM - 1) / BM, (a.K + BN - 1) / BN, split);
  dim3 block(WVM * WVN * 64);
  if (grid.y > 65535u || grid.z > 65535u) return fail(NITI_ERR_UNSUPPORTED, "conv: K=%d too large", a.K);
  static bool attr_set_of[kDeviceSlots][2] = {};   // function attributes are per device
  bool* const attr_set = attr_set_of[device_slot()];
  if (split > 1) {
    auto k = conv_mfma_kernel<WVM, WVN, WP, WC, STAGES, BK, true>;
    if (!attr_set[1]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return fail(NITI_ERR_LAUNCH, "conv: cannot reserve %zu bytes of LDS", lds);
      attr_set[1] = true;
    }
    hipLaunchKernelGGL(k, grid, block, lds, stream, a);
  } else {
    auto k = conv_mfma_kernel<WVM, WVN, WP, WC, STAGES, BK, false>;
    if (!attr_set[0]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
        return fail(NITI_ERR_LAUNCH, "conv: cannot reserve %zu bytes of LDS", lds);
      attr_set[0] = true;
    }
    hipLaunchKernelGGL(k, grid, block, lds, stream, a);
  }
  return check_launch("conv_mfma");
}

}  // namespace

bool conv_mfma_supported(const ConvArgs& a) {
  return a.R * a.S <= 32 && a.C % 16 == 0 && a.x_bytes < 0x7fffffffLL && a.w_bytes < 0x7fffffffLL &&
         a.y_bytes < 0x7fffffffLL;
}

int launch_conv_mfma(const ConvArgs& a, int split, hipStream_t stream) {
  const int force = a.tile_override;
  auto tiles = [&](int bm, int bn) { return static_cast<long long>((a.M + bm - 1) / bm) * ((a.K + bn - 1) / bn) * split; };
  // 128-byte reduction steps fetch whole cache lines of every pixel / filter row; they need each
  // step to stay inside one filter tap
  const bool wide = a.C % 128 == 0;
  int pick;
  if (force) pick = force;
  else if (wide) pick = tiles(256, 128) >= 224 ? 5 : 6;
  else if (a.K <= 128 && tiles(512, 128) >= 224) pick = 1;
  else if (tiles(256, 128) >= 224) pick = 3;
  else pick = 4;
  if ((pick == 5 || pick == 6) && !wide) pick = 4;
  switch (pick) {
    case 1: return launch_cfg<4, 2, 4, 2, 3, 64>(a, split, stream);   // 512 x 128, 8 wavefronts
    case 2: return launch_cfg<2, 4, 4, 2, 3, 64>(a, split, stream);   // 256 x 256, 8 wavefronts
    case 3: return launch_cfg<2, 2, 4, 2, 3, 64>(a, split, stream);   // 256 x 128, 4 wavefronts
    case 5: return launch_cfg<4, 2, 2, 2, 3, 128>(a, split, stream);  // 256 x 128 x 128, 8 wavefronts
    case 6: return launch_cfg<2, 2, 2, 2, 3, 128>(a, split, stream);  // 128 x 128 x 128, 4 wavefronts
    default: return launch_cfg<2, 2, 2, 2, 3, 64>(a, split, stream);  // 128 x 128, 4 wavefronts
  }
}

}  // namespace niti
