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
// v_mfma_i32_32x32x32_i8.  One halo buffer plus a 4-deep ring of filter taps keeps a workgroup
// under 80 KB of LDS and 128 VGPRs, so two workgroups share a compute unit: while one waits for its
// next halo slice, starts up or writes its results, the other one feeds the matrix cores.  The same
// kernel computes the data gradient when given the flipped / transposed filter arrangement
// (prepare kernel, mode 1).
//
// Requantising variant (kFused): the int32 sums never leave the registers.  Every workgroup publishes
// the largest magnitude of its tile in a slot of its own, waits until the slots of all workgroups of the
// launch are filled (they are all resident: the host refuses grids larger than the chip holds at once,
// and the wait is bounded by a wall-clock limit so that every wavefront exits whatever happens), derives
// the tensor-wide shift from the maximum over the slots and stores rounded int8.  Compared with the
// int32 store + separate requantisation pass this removes 8 of the 9 bytes moved per output element.
#include "common.h"
#include "requant_math.h"

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
  // requantising variant only
  int8_t* y8;         // [N,Q,Q,K] int8
  uint32_t* sync;     // word 0: max |sum| of the launch (output), word 1: set when the wait gave up,
                      // words kSyncSlot0..: one slot per workgroup, max + 1; all zero on entry
  long long y8_bytes;
  int target_bits, method, trunc, bw_mode;
  unsigned rq_flags;
  long long spin_limit;  // wall-clock ticks (100 MHz) the wait may last
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};
constexpr int kSyncSlot0 = 16;

// Q: image width = height; BR: output rows of one image per workgroup; NI: images per workgroup; BR*NI*Q == 256
template <int Q, int BR, int NI>
struct HGeom {
  static constexpr int RP = (Q + 2 + 15) / 16 * 16;
  static constexpr int HR = BR + 2;
  static constexpr int ACT_INSTR = NI * HR * (RP / 16);
  static constexpr int ACT_BYTES = NI * HR * RP * 64;
  static constexpr int ACT_LOADS = (ACT_INSTR + 7) / 8;  // per wavefront per slice
  static constexpr int W_BYTES = 128 * 64;               // one filter stage: one tap
  static constexpr int WSTAGES = 4;
  static constexpr int LDS_BYTES = ACT_BYTES + WSTAGES * W_BYTES + 1024;  // + dump slot
  static_assert(BR * NI * Q == 256, "a workgroup owns 256 output pixels");
};

template <int Q, int BR, int NI, bool kFused>
__global__ __launch_bounds__(512, 4) void conv3x3_halo_kernel(const HaloArgs a) {
  using G = HGeom<Q, BR, NI>;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const act_buf = smem;                         // ACT_BYTES
  int8_t* const w_buf = smem + G::ACT_BYTES;            // WSTAGES x 8 KB
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
  auto issue_act = [&](int cs) {
    int8_t* base = act_buf;
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
  // ---- filter staging: stage (cs, tap) is one contiguous 8 KB block; one KB per wavefront
  const int wstep_base = (kt * a.cslices) * 9 * G::W_BYTES + wave * 1024 + lane * 16;
  auto issue_w = [&](int step, int st) {  // step = cs * 9 + tap
    int8_t* dst = w_buf + st * G::W_BYTES + wave * 1024;
    const int off = wstep_base + step * G::W_BYTES;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS(dst), 16, off, 0, 0, 0);
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

  // ---- pipeline.  Per-wavefront load order: act(slice 0), W(0), W(1), W(2); inside step t: W(t+3); before
  // the first step of every later slice: act(slice).  All waits are derived from that order.
  // Every workgroup of a launch streams the same filter; integer sums do not depend on the order, so each
  // workgroup starts at its own channel slice and filter row and wraps around, which spreads the
  // simultaneous requests over the filter copy instead of piling them onto the same lines.
  const int nst = a.cslices * 9;
  const int cs0 = blockIdx.x % a.cslices;
  const int r0 = (blockIdx.x / a.cslices) % 3;
  auto slice_of = [&](int ci) { const int c = ci + cs0; return c >= a.cslices ? c - a.cslices : c; };
  auto tap_of = [&](int ti) {  // ti-th tap in this workgroup's order
    const int ri = ti / 3, s = ti - ri * 3;
    const int r = ri + r0 >= 3 ? ri + r0 - 3 : ri + r0;
    return r * 3 + s;
  };
  auto stage_of = [&](int t) { const int ci = t / 9; return slice_of(ci) * 9 + tap_of(t - ci * 9); };
  issue_act(slice_of(0));
  issue_w(stage_of(0), 0);
  if (1 < nst) issue_w(stage_of(1), 1);
  if (2 < nst) issue_w(stage_of(2), 2);
  for (int ci = 0; ci < a.cslices; ++ci) {
    if (ci > 0) {
      hc_sync();  // every wavefront has finished reading the previous slice
      issue_act(slice_of(ci));
    }
#pragma unroll
    for (int ti = 0; ti < 9; ++ti) {
      const int t = ci * 9 + ti;
      // younger than W(t): W(t+1), W(t+2); the halo slice issued just above is the youngest of all
      const int young = min(2, nst - 1 - t);
      if (ti == 0 && ci > 0) hc_wait_vmcnt<0>();
      else if (young == 2) hc_wait_vmcnt<2>();
      else if (young == 1) hc_wait_vmcnt<1>();
      else hc_wait_vmcnt<0>();
      hc_sync();
      if (t + 3 < nst) issue_w(stage_of(t + 3), (t + 3) % G::WSTAGES);
      const int tap = tap_of(ti);
      const int r = tap / 3, s = tap - r * 3;
      const int8_t* sw = w_buf + (t % G::WSTAGES) * G::W_BYTES;
      const int roff = r * G::RP * 64;
      int pa[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) pa[j] = (s == 0 ? p_addr[j][0] : (s == 1 ? p_addr[j][1] : p_addr[j][2])) + roff;
      v4i wf[2][2], pf[2][2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
        for (int i = 0; i < 2; ++i) wf[kk][i] = *reinterpret_cast<const v4i*>(sw + (w_addr[i] ^ (kk << 5)));
#pragma unroll
        for (int j = 0; j < 2; ++j) pf[kk][j] = *reinterpret_cast<const v4i*>(act_buf + (pa[j] ^ (kk << 5)));
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[kk][i], pf[kk][j], acc[i][j], 0, 0, 0);
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
  // The fp32 round trip is the identity up to 2^24, so it is applied (wavefront-uniformly) only beyond; it is
  // monotonic and odd, so the range after it follows from the extreme values alone, and the sums themselves
  // are converted where they are consumed below instead of in a second copy of the accumulators.
  bool rt = false;
  if (roundtrip) rt = wave_max_u32(max(static_cast<uint32_t>(vmax), 0u - static_cast<uint32_t>(vmin))) > (1u << 24);
  if (rt) {
    vmax = f32_roundtrip(vmax);
    vmin = f32_roundtrip(vmin);
  }
  const uint32_t lmax = max(static_cast<uint32_t>(vmax), 0u - static_cast<uint32_t>(vmin));
  const long long total_pix = static_cast<long long>(a.N) * Q * Q;
  if constexpr (!kFused) {
  hc_sync();  // all wavefronts are done with the tiles: reuse LDS as per-wavefront transposition patches
  constexpr int ROWB = 32 * 4 + 16;  // one 32-channel tile row of int32, padded
  int8_t* patch = smem + wave * (32 * ROWB);
  const int rrow = lane >> 3, rcol = lane & 7;  // 8 lanes x 16 bytes = one 32-channel row
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int mrow = pixbase + wp_ * 64 + j * 32 + rrow;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        v4i v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        if (rt) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = f32_roundtrip(v[e]);
        }
        *reinterpret_cast<v4i*>(patch + lr * ROWB + (g * 8 + lk * 4) * 4) = v;
      }
      // same wavefront reads back what it wrote: LDS operations of one wavefront complete in order
      const int ch = kt * 128 + wc * 64 + i * 32 + rcol * 4;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const v4i v = *reinterpret_cast<const v4i*>(patch + (t * 8 + rrow) * ROWB + rcol * 16);
        const int m = mrow + t * 8;
        const int off = (m < total_pix && ch < a.K) ? (m * a.K + ch) * 4 : kOob;
        __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0);
      }
    }
  }
  if (a.absmax != nullptr) fold_absmax(a.absmax, lmax);
  } else {
  // ---- tensor-wide range: workgroup maximum -> own slot -> wait for all slots -> maximum over the slots
  uint32_t* const red = reinterpret_cast<uint32_t*>(dump);  // behind the tiles, clear of the patches below
  const uint32_t wmax = wave_max_u32(lmax);
  __syncthreads();  // the tiles are dead from here on
  if (lane == 0) red[wave] = wmax;
  __syncthreads();
  if (wave == 0) {
    uint32_t bmax = lane < 8 ? red[lane] : 0u;
    bmax = wave_max_u32(bmax);
    const int nb = gridDim.x * gridDim.y;
    const int b = blockIdx.y * gridDim.x + blockIdx.x;
    uint32_t* const slots = a.sync + kSyncSlot0;
    if (lane == 0) __hip_atomic_store(&slots[b], bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const long long t0 = wall_clock64();
    uint32_t g = 0;
    for (;;) {
      bool ok = true;
      g = 0;
      for (int i = lane; i < nb; i += 64) {
        const uint32_t v = __hip_atomic_load(&slots[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = ok && v != 0u;
        g = v > g ? v : g;
      }
      if (__all(ok)) break;
      if (wall_clock64() - t0 > a.spin_limit) {  // not every workgroup showed up: flag it and leave anyway
        if (lane == 0) __hip_atomic_store(&a.sync[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
    g = wave_max_u32(g);
    if (lane == 0) red[8] = g != 0u ? g - 1u : 0u;
  }
  __syncthreads();
  const uint32_t gmax = red[8];
  const int shift = bitwidth_of(gmax, a.bw_mode) - a.target_bits;
  if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) {
    const int sh = shift > 0 ? shift : 0;
    a.sync[0] = gmax;
    if (a.shift_out != nullptr) *a.shift_out = sh;
    if (a.exp_out != nullptr)
      *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
  }
  // ---- round, pack four channels per dword, transpose through a per-wavefront patch, store 16-byte pieces
  const bool trunc = a.trunc != 0;
  const bool relu = (a.rq_flags & NITI_RQ_RELU) != 0;
  const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
  constexpr int PROW = 64 + 16;  // 64 channels of one pixel, padded
  int8_t* patch = smem + wave * (64 * PROW);
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int x = acc[i][j][4 * g + e];
          if (rt) x = f32_roundtrip(x);
          int r;
          if (shift >= 1) r = psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, shift, trunc) : round_one32<NITI_ROUND_NEAREST>(x, shift, trunc);
          else r = wrap_to_i8(x);
          if (relu && r < 0) r = 0;
          packed |= (static_cast<uint32_t>(r) & 0xFFu) << (8 * e);
        }
        *reinterpret_cast<uint32_t*>(patch + (j * 32 + lr) * PROW + (i * 8 + 2 * g + lk) * 4) = packed;
      }
  // same wavefront reads back what it wrote: LDS operations of one wavefront complete in order
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y8, 0, a.y8_bytes, 0x00020000);
  const int prow = lane >> 2, piece = lane & 3;
  const int ch = kt * 128 + wc * 64 + piece * 16;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int pl = t * 16 + prow;
    const v4i v = *reinterpret_cast<const v4i*>(patch + pl * PROW + piece * 16);
    const int m = pixbase + wp_ * 64 + pl;
    const int off = (m < total_pix && ch < a.K) ? m * a.K + ch : kOob;
    __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 0);
  }
  }
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

template <int Q, int BR, int NI, bool kFused>
int launch_halo(const HaloArgs& a, hipStream_t stream) {
  using G = HGeom<Q, BR, NI>;
  constexpr size_t lds = G::LDS_BYTES;
  static_assert(lds <= 160 * 1024, "tiles must fit in LDS");
  static_assert(8 * 32 * (32 * 4 + 16) <= G::ACT_BYTES + G::WSTAGES * G::W_BYTES, "epilogue patches must fit in LDS");
  static_assert(8 * 64 * (64 + 16) <= G::ACT_BYTES + G::WSTAGES * G::W_BYTES, "int8 patches must stay clear of the reduction words");
  static_assert(2 * lds <= 160 * 1024, "two workgroups per compute unit");
  auto k = conv3x3_halo_kernel<Q, BR, NI, kFused>;
  static bool attr_set = false;
  static int resident = 0;  // workgroups the device holds at once
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "conv3x3_halo: cannot reserve %zu bytes of LDS", lds);
    if (kFused) {
      int dev = 0, cus = 0, per_cu = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
          hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(k), 512, lds) != hipSuccess)
        return fail(NITI_ERR_LAUNCH, "conv3x3_halo: cannot query occupancy");
      resident = cus * per_cu;
    }
    attr_set = true;
  }
  const long long pix = static_cast<long long>(a.N) * Q * Q;
  dim3 grid(static_cast<unsigned>((pix + 255) / 256), (a.K + 127) / 128);
  if (kFused && static_cast<long long>(grid.x) * grid.y > resident)
    return fail(NITI_ERR_UNSUPPORTED, "conv3x3_halo: %u workgroups do not fit on the device at once (%d)", grid.x * grid.y, resident);
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

static void fill_common(HaloArgs& a, const int8_t* x, const int8_t* wp, int N, int H, int C, int K, unsigned flags) {
  a = HaloArgs{};
  a.x = x;
  a.wp = wp;
  a.N = N;
  a.C = C;
  a.K = K;
  a.cslices = (C + 63) / 64;
  a.x_bytes = static_cast<long long>(N) * H * H * C;
  a.wp_bytes = static_cast<long long>(conv3x3_halo_filter_bytes(C, K));
  a.flags = flags;
}

int launch_conv3x3_halo(const int8_t* x, const int8_t* wp, int32_t* y, int N, int H, int C, int K, unsigned flags,
                        uint32_t* absmax, hipStream_t stream) {
  HaloArgs a;
  fill_common(a, x, wp, N, H, C, K, flags);
  a.y = y;
  a.absmax = absmax;
  a.y_bytes = static_cast<long long>(N) * H * H * K * 4;
  if (H == 32) return launch_halo<32, 8, 1, false>(a, stream);
  if (H == 16) return launch_halo<16, 16, 1, false>(a, stream);
  return launch_halo<8, 8, 4, false>(a, stream);
}

// Workgroups of a launch of the requantising variant (= sync slots), or 0 when the variant cannot run the shape.
int conv3x3_halo_requant_blocks(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (!conv3x3_halo_supported(N, H, W, C, K, R, S, stride, pad) || K % 16 != 0) return 0;
  const long long nb = (static_cast<long long>(N) * H * W / 256) * ((K + 127) / 128);
  return nb <= 2048 ? static_cast<int>(nb) : 0;  // the device check happens at launch; this bounds the workspace
}

size_t conv3x3_halo_sync_words(int blocks) { return static_cast<size_t>(kSyncSlot0 + (blocks + 15) / 16 * 16); }

int launch_conv3x3_halo_requant(const int8_t* x, const int8_t* wp, int8_t* y8, int N, int H, int C, int K, unsigned flags,
                                uint32_t* sync, const RequantSpec& rq, hipStream_t stream) {
  HaloArgs a;
  fill_common(a, x, wp, N, H, C, K, flags);
  a.y8 = y8;
  a.sync = sync;
  a.y8_bytes = static_cast<long long>(N) * H * H * K;
  a.target_bits = rq.target_bits;
  a.method = rq.method;
  a.trunc = rq.trunc;
  a.bw_mode = rq.bw_mode;
  a.rq_flags = rq.flags;
  a.spin_limit = rq.spin_limit;
  a.shift_out = rq.shift_out;
  a.exp_a = rq.exp_a;
  a.exp_b = rq.exp_b;
  a.exp_out = rq.exp_out;
  if (H == 32) return launch_halo<32, 8, 1, true>(a, stream);
  if (H == 16) return launch_halo<16, 16, 1, true>(a, stream);
  return launch_halo<8, 8, 4, true>(a, stream);
}

}  // namespace niti
