// int8 3x3 / stride 1 / pad 1 convolution forward on the gfx950 matrix cores with the activation
// halo tile resident in LDS ("read every activation once, not once per filter tap").
//
// The plain implicit GEMM (conv_mfma.hip) fetches each activation nine times and each filter row
// once per pixel tile through L2; L2 sustains about 30 bytes/clock/CU next to running MFMAs while
// that kernel needs 48-64.  Here a workgroup owns 256 consecutive output pixels (whole rows of an
// image, or whole small images) x 128 output channels and walks over the input channels in slices
// of 64: per slice it stages the activation rows with their one-pixel halo once (about 35 KB,
// out-of-image positions read as zero through an out-of-range buffer offset) and serves all nine
// taps from that tile; the filter streams row by row (24 KB per stage) from a pre-arranged copy whose
// memory image is exactly the swizzled LDS tile, so every load instruction moves one contiguous KB.
// About 23 bytes/clock/CU at MFMA peak.
//
// 8 wavefronts (4 pixel groups x 2 channel halves), each 64 pixels x 64 channels = 2x2 tiles of
// v_mfma_i32_32x32x32_i8.  Halo slices are double buffered, filter stages run through a 3-deep
// ring of filter rows (three taps each); one s_barrier per filter row, LDS fragment reads
// software-pipelined one sub-step ahead of the MFMAs.  The same kernel computes the data gradient when given the
// flipped / transposed filter arrangement (prepare kernel, mode 1).
#include "common.h"

namespace niti {
namespace {

#define NITI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
constexpr int kOob = -1;

template <int N>
__device__ inline void hc_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | 0x0F70);
}
__device__ inline void hc_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

struct HaloArgs {
  const int8_t* x;    // [N,Q,Q,C]
  const int8_t* wp;   // prepared filter: [ktiles][cslices][9][128][64], rows XOR-swizzled
  int32_t* y;         // [N,Q,Q,K]
  uint32_t* absmax;
  int N, C, K;
  int cslices;        // ceil(C / 64)
  long long x_bytes, wp_bytes, y_bytes;
  unsigned flags;
};

// Q: image width = height; BR: output rows of one image per workgroup; NI: images per workgroup; BR*NI*Q == 256
template <int Q, int BR, int NI>
struct HGeom {
  static constexpr int RP = (Q + 2 + 15) / 16 * 16;
  static constexpr int HR = BR + 2;
  static constexpr int ACT_INSTR = NI * HR * (RP / 16);
  static constexpr int ACT_BYTES = NI * HR * RP * 64;
  static constexpr int ACT_LOADS = (ACT_INSTR + 7) / 8;  // per wavefront per slice
  static constexpr int W_BYTES = 3 * 128 * 64;           // one filter stage: the three taps of a filter row
  static constexpr int WSTAGES = 3;
  static constexpr int LDS_BYTES = 2 * ACT_BYTES + WSTAGES * W_BYTES + 1024;  // + dump slot
  static_assert(BR * NI * Q == 256, "a workgroup owns 256 output pixels");
};

template <int Q, int BR, int NI>
__global__ __launch_bounds__(512, 1) void conv3x3_halo_kernel(const HaloArgs a) {
  using G = HGeom<Q, BR, NI>;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const act_buf = smem;                         // 2 x ACT_BYTES
  int8_t* const w_buf = smem + 2 * G::ACT_BYTES;        // WSTAGES x 8 KB
  int8_t* const dump = w_buf + G::WSTAGES * G::W_BYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pixbase = blockIdx.x * 256;  // first output pixel of this workgroup in [N*Q*Q]
  const int kt = blockIdx.y;
  const int n0 = pixbase / (Q * Q);
  const int p0 = (pixbase - n0 * (Q * Q)) / Q;

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.wp), 0, a.wp_bytes, 0x00020000);

  // ---- activation staging: an instruction fills 16 pixel slots x 64 bytes; lane -> (slot lane/4, piece lane%4)
  int act_off[G::ACT_LOADS];  // byte offset for channel slice 0, or kOob
  int act_dst[G::ACT_LOADS];  // LDS offset of the instruction's KB inside the halo tile, or -1 (dump)
  const int ab = (n0 * Q + p0) * Q * a.C;
#pragma unroll
  for (int i = 0; i < G::ACT_LOADS; ++i) {
    const int idx = wave + 8 * i;
    int off = kOob, dst = -1;
    if (idx < G::ACT_INSTR) {
      const int ni = idx / (G::HR * (G::RP / 16));
      const int rem = idx - ni * (G::HR * (G::RP / 16));
      const int h = rem / (G::RP / 16);
      const int wg = rem - h * (G::RP / 16);
      const int w = wg * 16 + (lane >> 2);
      const int piece = (lane & 3) ^ ((w >> 2) & 3);
      const int ih = p0 + h - 1, iw = w - 1;
      dst = ((ni * G::HR + h) * G::RP + wg * 16) * 64;
      if (n0 + ni < a.N && ih >= 0 && ih < Q && iw >= 0 && iw < Q && w < Q + 2)
        off = ab + ((ni * Q + (h - 1)) * Q + iw) * a.C + piece * 16;
    }
    act_off[i] = off;
    act_dst[i] = dst;
  }
  auto issue_act = [&](int cs, int buf) {
    int8_t* base = act_buf + buf * G::ACT_BYTES;
#pragma unroll
    for (int i = 0; i < G::ACT_LOADS; ++i) {
      // channel range check: the 16 bytes at slice offset cs*64 + piece*16 must lie inside C
      int off = act_off[i];
      if (off != kOob) {
        const int w = ((wave + 8 * i) % (G::RP / 16)) * 16 + (lane >> 2);
        const int piece = (lane & 3) ^ ((w >> 2) & 3);
        off = (cs * 64 + piece * 16 < a.C) ? off + cs * 64 : kOob;
      }
      int8_t* dst = act_dst[i] >= 0 ? base + act_dst[i] : dump;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, NITI_LDS(dst), 16, off, 0, 0, 0);
    }
  };
  // ---- filter staging: stage (cs, r) is one contiguous 24 KB block (three taps); three KB per wavefront
  const int wstep_base = (kt * a.cslices) * 3 * G::W_BYTES + wave * 1024 + lane * 16;
  auto issue_w = [&](int step, int st) {  // step = cs * 3 + r
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      int8_t* dst = w_buf + st * G::W_BYTES + s * 8192 + wave * 1024;
      const int off = wstep_base + step * G::W_BYTES + s * 8192;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS(dst), 16, off, 0, 0, 0);
    }
  };

  // ---- fragment addressing
  const int wp_ = wave & 3;   // 64-pixel group
  const int wc = wave >> 2;   // 64-channel half
  const int lr = lane & 31, lk = lane >> 5;
  int w_addr[2];              // filter rows of this lane, reduction half 0 (the other half is ^32)
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = wc * 64 + i * 32 + lr;
    w_addr[i] = row * 64 + ((lk ^ ((row >> 2) & 3)) << 4);
  }
  int p_addr[2][3];           // [pixel tile][s]: halo slot of this lane's pixel for filter column s, filter row 0
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int pix = wp_ * 64 + j * 32 + lr;       // output pixel inside the workgroup's 256
    const int prow = pix / Q, pw = pix % Q;        // row inside the workgroup's rows, column
    const int hrow = (prow / BR) * G::HR + (prow % BR);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      const int w = pw + s;
      p_addr[j][s] = (hrow * G::RP + w) * 64 + ((lk ^ ((w >> 2) & 3)) << 4);
    }
  }

  v16i acc[2][2];  // [channel tile][pixel tile]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // ---- pipeline.  Per-wavefront load order: act(0), W(0), W(1), then inside stage t: W(t+2) and, at the
  // first stage of every slice, act(next slice).  All waits are derived from that order.
  // Every workgroup of a launch streams the same filter; started together they would all pull the same
  // 24 KB through the same few L2 channels at the same time.  Integer sums do not depend on the order,
  // so each workgroup starts at its own channel slice and filter row and wraps around.
  const int nst = a.cslices * 3;
  const int cs0 = blockIdx.x % a.cslices;
  const int r0 = (blockIdx.x / a.cslices) % 3;
  auto slice_of = [&](int ci) { const int c = ci + cs0; return c >= a.cslices ? c - a.cslices : c; };
  auto stage_of = [&](int t) {  // t-th stage in this workgroup's order -> index in the filter copy
    const int ci = t / 3, ri = t - ci * 3;
    const int r = ri + r0 >= 3 ? ri + r0 - 3 : ri + r0;
    return slice_of(ci) * 3 + r;
  };
  issue_act(slice_of(0), 0);
  issue_w(stage_of(0), 0);
  if (1 < nst) issue_w(stage_of(1), 1);
  for (int ci = 0; ci < a.cslices; ++ci) {
    const int8_t* sact = act_buf + (ci & 1) * G::ACT_BYTES;
#pragma unroll
    for (int ri = 0; ri < 3; ++ri) {
      const int t = ci * 3 + ri;
      // younger than W(t) and possibly still in flight: W(t+1); act(next slice), issued at ri == 0 after W(t+2)
      const bool young_w = t + 1 < nst;
      const bool young_act = ri >= 1 && ci + 1 < a.cslices;
      if (young_act) {
        if (young_w) hc_wait_vmcnt<3 + G::ACT_LOADS>();
        else hc_wait_vmcnt<G::ACT_LOADS>();
      } else {
        if (young_w) hc_wait_vmcnt<3>();
        else hc_wait_vmcnt<0>();
      }
      hc_sync();
      if (t + 2 < nst) issue_w(stage_of(t + 2), (t + 2) % G::WSTAGES);
      if (ri == 0 && ci + 1 < a.cslices) issue_act(slice_of(ci + 1), (ci + 1) & 1);
      const int r = ri + r0 >= 3 ? ri + r0 - 3 : ri + r0;
      const int8_t* sw = w_buf + (t % G::WSTAGES) * G::W_BYTES;
      const int roff = r * G::RP * 64;
      // six sub-steps (three taps x two 32-byte reduction halves); fragments of sub-step i+1 are
      // fetched from LDS before the MFMAs of sub-step i are issued
      v4i wf[2][2], pf[2][2];
      auto fetch = [&](int sub, int slot) {
        const int s = sub >> 1, kk = sub & 1;
#pragma unroll
        for (int i = 0; i < 2; ++i)
          wf[slot][i] = *reinterpret_cast<const v4i*>(sw + s * 8192 + (w_addr[i] ^ (kk << 5)));
#pragma unroll
        for (int j = 0; j < 2; ++j)
          pf[slot][j] = *reinterpret_cast<const v4i*>(sact + ((p_addr[j][s] ^ (kk << 5)) + roff));
      };
      fetch(0, 0);
#pragma unroll
      for (int sub = 0; sub < 6; ++sub) {
        if (sub + 1 < 6) fetch(sub + 1, (sub + 1) & 1);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[sub & 1][i], pf[sub & 1][j], acc[i][j], 0, 0, 0);
      }
    }
  }

  // ---- epilogue: acc[i][j][4g+e] = channel kt*128+wc*64+i*32+8g+4*lk+e of pixel pixbase+wp_*64+j*32+lr
  const bool roundtrip = (a.flags & NITI_EPI_F32_ROUNDTRIP) != 0;
  int vmax = 0, vmin = 0;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        vmax = max(vmax, max(acc[i][j][e], acc[i][j][e + 1]));
        vmin = min(vmin, min(acc[i][j][e], acc[i][j][e + 1]));
      }
  uint32_t lmax = max(static_cast<uint32_t>(vmax), 0u - static_cast<uint32_t>(vmin));
  if (roundtrip && wave_max_u32(lmax) > (1u << 24)) {
    lmax = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int t = f32_roundtrip(acc[i][j][e]);
          acc[i][j][e] = t;
          const uint32_t u = uabs(t);
          lmax = u > lmax ? u : lmax;
        }
  }
  hc_sync();  // all wavefronts are done with the tiles: reuse LDS as per-wavefront transposition patches
  constexpr int ROWB = 64 * 4 + 16;
  int8_t* patch = smem + wave * (32 * ROWB);
  const int rrow = lane >> 4, rcol = lane & 15;  // 16 lanes x 16 bytes = one 64-channel row
  const int ch = kt * 128 + wc * 64 + rcol * 4;
  const long long total_pix = static_cast<long long>(a.N) * Q * Q;
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v4i v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        *reinterpret_cast<v4i*>(patch + lr * ROWB + (i * 32 + g * 8 + lk * 4) * 4) = v;
      }
    const int mrow = pixbase + wp_ * 64 + j * 32 + rrow;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const v4i v = *reinterpret_cast<const v4i*>(patch + (t * 4 + rrow) * ROWB + rcol * 16);
      const int m = mrow + t * 4;
      const int off = (m < total_pix && ch < a.K) ? (m * a.K + ch) * 4 : kOob;
      __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0);
    }
  }
  if (a.absmax != nullptr) fold_absmax(a.absmax, lmax);
}

// Filter arrangement for the kernel above.  mode 0 (forward): F(k, tap, c) = w[k][tap][c], w is [K][9][C].
// mode 1 (data gradient): the roles of the channel dimensions swap and the taps flip:
// F(k', tap, c') = w[c'][8 - tap][k'], with k' < C and c' < K of the original filter.
// dst[kt][cs][tap][row][piece ^ ((row >> 2) & 3)][16] = F(kt*128 + row, tap, cs*64 + piece*16 ..), zero outside.
__global__ __launch_bounds__(256) void halo_filter_prepare_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ dst,
                                                                  int kout, int cin, int mode, int64_t total) {
  const int cslices = (cin + 63) / 64;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int b = static_cast<int>(i & 15);
    const int ppos = static_cast<int>((i >> 4) & 3);
    const int row = static_cast<int>((i >> 6) & 127);
    int64_t t = i >> 13;
    const int tap = static_cast<int>(t % 9);
    t /= 9;
    const int cs = static_cast<int>(t % cslices);
    const int kt = static_cast<int>(t / cslices);
    const int piece = ppos ^ ((row >> 2) & 3);
    const int k = kt * 128 + row;
    const int c = cs * 64 + piece * 16 + b;
    int8_t v = 0;
    if (k < kout && c < cin) {
      if (mode == 0) v = w[(static_cast<int64_t>(k) * 9 + tap) * cin + c];
      else v = w[(static_cast<int64_t>(c) * 9 + (8 - tap)) * kout + k];
    }
    dst[i] = v;
  }
}

template <int Q, int BR, int NI>
int launch_halo(const HaloArgs& a, hipStream_t stream) {
  using G = HGeom<Q, BR, NI>;
  constexpr size_t lds = G::LDS_BYTES;
  static_assert(lds <= 160 * 1024, "tiles must fit in LDS");
  static_assert(8 * 32 * (64 * 4 + 16) <= lds, "epilogue patches must fit in LDS");
  auto k = conv3x3_halo_kernel<Q, BR, NI>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "conv3x3_halo: cannot reserve %zu bytes of LDS", lds);
    attr_set = true;
  }
  const long long pix = static_cast<long long>(a.N) * Q * Q;
  dim3 grid(static_cast<unsigned>((pix + 255) / 256), (a.K + 127) / 128);
  hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, a);
  return check_launch("conv3x3_halo");
}

}  // namespace

bool conv3x3_halo_supported(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (R != 3 || S != 3 || stride != 1 || pad != 1 || H != W) return false;
  if (H != 8 && H != 16 && H != 32) return false;
  if (C % 16 != 0 || K % 4 != 0) return false;
  const long long pix = static_cast<long long>(N) * H * W;
  if (pix % 256 != 0) return false;  // workgroups own whole rows / whole images
  if (pix * C >= 0x7fffffffLL || pix * K * 4 >= 0x7fffffffLL) return false;
  return true;
}

size_t conv3x3_halo_filter_bytes(int C, int K) {
  return static_cast<size_t>((K + 127) / 128) * ((C + 63) / 64) * 9 * 128 * 64;
}

// w: [K][3][3][C] (mode 0) or, for the data gradient (mode 1), the forward filter [Kf][3][3][Cf] with kout = Cf, cin = Kf
int launch_halo_filter_prepare(const int8_t* w, int8_t* dst, int kout, int cin, int mode, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(conv3x3_halo_filter_bytes(cin, kout));
  int64_t g = (total + 255) / 256;
  if (g > 4096) g = 4096;
  hipLaunchKernelGGL(halo_filter_prepare_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0, stream, w, dst, kout, cin, mode, total);
  return check_launch("halo_filter_prepare");
}

int launch_conv3x3_halo(const int8_t* x, const int8_t* wp, int32_t* y, int N, int H, int C, int K, unsigned flags,
                        uint32_t* absmax, hipStream_t stream) {
  HaloArgs a;
  a.x = x;
  a.wp = wp;
  a.y = y;
  a.absmax = absmax;
  a.N = N;
  a.C = C;
  a.K = K;
  a.cslices = (C + 63) / 64;
  a.x_bytes = static_cast<long long>(N) * H * H * C;
  a.wp_bytes = static_cast<long long>(conv3x3_halo_filter_bytes(C, K));
  a.y_bytes = static_cast<long long>(N) * H * H * K * 4;
  a.flags = flags;
  if (H == 32) return launch_halo<32, 8, 1>(a, stream);
  if (H == 16) return launch_halo<16, 16, 1>(a, stream);
  return launch_halo<8, 8, 4>(a, stream);
}

}  // namespace niti
