// Weight gradient + grad_calc + weight update of a 3x3 / stride-1 / pad-1 convolution on 4 x 4 and 2 x 2 maps as ONE
// launch (ti_torch.py:430-432, :16-21).
//
// The last layers of a deep network have few pixels and many weights: 512 -> 512 channels on 2 x 2 maps at batch 256
// are 1024 pixels against 2.4 M gradient elements.  The general kernel pair (wgrad3x3.hip: partial sums of ~256
// workgroups through memory, then a finishing launch) spends 22-29 us there on 5-19 GOP, almost all of it in the two
// launches, the cold first stage and 2 x 37.7 MB of partial sums.  Here nothing is split: a workgroup owns 32 output
// channels x 32 input channels x 9 taps and walks over ALL pixels, so its sums are final and the same launch exchanges
// the range, rounds and applies w = clip(w - g) (and keeps the forward pass's kernel-ready filter copy in step).
//
// A workgroup is 9 wavefronts, one per tap.  Per stage of 256 pixels it stages the 32-channel slice of the activations
// and of the errors in their natural [pixel][32 bytes] layout (buffer_load ... lds, ring of four stages); fragments are
// transposing LDS reads (ds_read_b64_tr_b8: every lane names an 8-byte piece of a pixel).  Maps this small lie whole
// inside every reduction step of 32 pixels, so a tap is nothing but another pixel for each lane's address - or, where
// the neighbour falls outside the image, a row of zeros.
#include "common.h"
#include "lds_asm.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kWsChunk = 256;                       // pixels per stage
constexpr int kWsStages = 4;
constexpr int kWsTile = kWsChunk * 32;              // bytes of one operand tile
constexpr int kWsStageBytes = 2 * kWsTile;          // activations, then errors
constexpr int kWsZeroAt = kWsStages * kWsStageBytes;
constexpr int kWsLdsBytes = kWsZeroAt + 64;
constexpr int kWsSlot0 = 16;                        // the finishing kernel's sync layout: slots from word 16
constexpr int kWsLoads = 2;                         // loads per wavefront (0..7) and stage

struct WsArgs {
  const int8_t* act;   // [pixels][C]
  const int8_t* err;   // [pixels][K]
  int8_t* w;           // [K][9][C], updated in place
  int8_t* g8;          // optional rounded gradient
  int32_t* dw;         // optional int32 gradient
  int8_t* wprep;       // optional kernel-ready forward filter copy
  uint32_t* sync;
  int pixels, C, K;
  long long act_bytes, err_bytes;
  int roundtrip, target_bits, method, trunc, bw_mode;
  long long spin_limit;
  uint32_t* sticky;
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};

template <int N>
__device__ inline void ws_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | 0x0F70);
}
__device__ inline void ws_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int Q>
__global__ __launch_bounds__(576) void wgrad_small_kernel(const WsArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  __shared__ uint32_t wmax[9];
  __shared__ uint32_t gshare;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tap = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront = filter tap
  const int c0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
  const int block = blockIdx.y * gridDim.x + blockIdx.x, nblocks = gridDim.x * gridDim.y;
  if (tid < 16) reinterpret_cast<uint32_t*>(smem + kWsZeroAt)[tid] = 0u;

  const __amdgpu_buffer_rsrc_t ract = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.act), 0, a.act_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rerr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.err), 0, a.err_bytes, 0x00020000);
  // staging: wavefront w < 8 fills pixels 32 w .. 32 w + 31 of both tiles; lane -> (pixel lane / 2, 16-byte half lane % 2)
  const int spix = tap * 32 + (lane >> 1);
  const int shalf = (lane & 1) * 16;
  auto issue = [&](int chunk, int st) {
    if (tap < 8) {
      const int m = chunk * kWsChunk + spix;
      const int xo = m < a.pixels ? m * a.C + c0 + shalf : -1;   // beyond the tensor: zeros
      const int eo = m < a.pixels ? m * a.K + k0 + shalf : -1;
      int8_t* const dst = smem + st * kWsStageBytes + tap * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ract, NITI_LDS(dst), 16, xo, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rerr, NITI_LDS(dst + kWsTile), 16, eo, 0, 0, 0);
    }
  };

  // fragment addressing: the lane names pixel frag (first read) and frag + 8 (second read) of a 32-pixel step and the
  // 8-byte column fo of its 32 channels
  const int j = lane & 15, gg = (lane >> 4) & 1, lk = lane >> 5;
  const int frag = lk * 16 + (j >> 1);
  const int fo = gg * 16 + 8 * (j & 1);
  const int dy = tap / 3 - 1, dx = tap % 3 - 1;
  unsigned x_off[2], x_step[2];   // activation piece of the tap's neighbour pixel, or the zero row
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int s = frag + 8 * h;
    const int pi = s % (Q * Q);
    const int p = pi / Q + dy, q = pi % Q + dx;
    const bool inside = p >= 0 && p < Q && q >= 0 && q < Q;
    x_off[h] = inside ? static_cast<unsigned>((s + dy * Q + dx) * 32 + fo) : static_cast<unsigned>(kWsZeroAt + fo);
    x_step[h] = inside ? 1024u : 0u;
  }
  const unsigned lds0 = lds_addr(smem);
  const unsigned e_off = static_cast<unsigned>(kWsTile + frag * 32 + fo);

  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;

  const int nchunks = (a.pixels + kWsChunk - 1) / kWsChunk;
#pragma unroll
  for (int s = 0; s < kWsStages - 1; ++s)
    if (s < nchunks) issue(s, s);
  for (int it = 0; it < nchunks; ++it) {
    if (it + kWsStages - 2 < nchunks) ws_wait_vmcnt<(kWsStages - 2) * kWsLoads>();
    else ws_wait_vmcnt<0>();
    ws_sync();
    if (it + kWsStages - 1 < nchunks) issue(it + kWsStages - 1, (it + kWsStages - 1) % kWsStages);
    const unsigned sbase = lds0 + static_cast<unsigned>((it % kWsStages) * kWsStageBytes);
    // an invalid neighbour reads the zero row, which is not part of a stage
    const unsigned xa0 = x_step[0] != 0u ? sbase + x_off[0] : lds0 + x_off[0];
    const unsigned xa1 = x_step[1] != 0u ? sbase + x_off[1] : lds0 + x_off[1];
    const unsigned eb = sbase + e_off;
    v2i alo[2], ahi[2], blo[2], bhi[2];
    auto request = [&](auto ksc) {
      constexpr int ks = decltype(ksc)::value;
      alo[ks & 1] = lds_read_tr8<0>(xa0 + ks * x_step[0]);
      ahi[ks & 1] = lds_read_tr8<0>(xa1 + ks * x_step[1]);
      blo[ks & 1] = lds_read_tr8<ks * 1024>(eb);
      bhi[ks & 1] = lds_read_tr8<ks * 1024 + 256>(eb);
    };
    request(std::integral_constant<int, 0>{});
    static_for<8>([&](auto ksc) {
      constexpr int ks = decltype(ksc)::value;
      if constexpr (ks + 1 < 8) request(std::integral_constant<int, ks + 1>{});
      lds_settle<(ks + 1 < 8) ? 4 : 0>();
      const v4i fa = lds_landed(alo[ks & 1], ahi[ks & 1]);
      const v4i fb = lds_landed(blo[ks & 1], bhi[ks & 1]);
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);   // the next step's requests and wait stay behind this product
    });
  }

  // ---- the sums are final: element 4 g + e of a lane is input channel c0 + 8 g + 4 (lane / 32) + e of output channel
  // k0 + lane % 32, tap = wavefront
  uint32_t lmax = 0;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    if (a.roundtrip) acc[e] = f32_roundtrip(acc[e]);
    const uint32_t u = uabs(acc[e]);
    lmax = u > lmax ? u : lmax;
  }
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[tap] = lmax;
  const int k = k0 + (lane & 31);
  const uint32_t row_base = static_cast<uint32_t>((k * 9 + tap) * a.C + c0 + 4 * lk);   // element index of the lane's first weight
  uint32_t wold[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) wold[g] = *reinterpret_cast<const uint32_t*>(a.w + row_base + 8 * g);   // in flight during the exchange
  __syncthreads();
  if (tap == 0) {
    uint32_t bmax = lane < 9 ? wmax[lane] : 0u;
    bmax = wave_max_u32(bmax);
    uint32_t* const slots = a.sync + kWsSlot0;
    if (lane == 0) __hip_atomic_store(slot_word(slots, block), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t g = wait_slots(slots, nblocks, a.spin_limit, &a.sync[1], a.sticky);
    if (lane == 0) gshare = g != 0u ? g - 1u : 0u;
  }
  __syncthreads();
  const uint32_t gmax = gshare;
  const int shift = max(bitwidth_of(gmax, a.bw_mode) - a.target_bits, 0);
  if (block == 0 && tid == 0) {
    a.sync[0] = gmax;
    if (a.shift_out != nullptr) *a.shift_out = shift;
    if (a.exp_out != nullptr) *a.exp_out = shift + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
  }
  const bool trunc = a.trunc != 0, psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    int r[4];
    uint32_t wnew = 0, gp = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int s = acc[4 * g + e];
      if (shift >= 1) r[e] = psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(s, shift, trunc) : round_one32<NITI_ROUND_NEAREST>(s, shift, trunc);
      else r[e] = wrap_to_i8(s);
      const int wo = static_cast<int>(static_cast<int8_t>((wold[g] >> (8 * e)) & 0xFFu));
      wnew |= (static_cast<uint32_t>(clip127(wo - r[e])) & 0xFFu) << (8 * e);
      gp |= (static_cast<uint32_t>(r[e]) & 0xFFu) << (8 * e);
    }
    const uint32_t at = row_base + 8 * g;
    *reinterpret_cast<uint32_t*>(a.w + at) = wnew;
    if (a.g8 != nullptr) *reinterpret_cast<uint32_t*>(a.g8 + at) = gp;
    if (a.dw != nullptr) *reinterpret_cast<v4i*>(a.dw + at) = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    if (a.wprep != nullptr) {
      // [64-channel group][32-channel slice][tap][64 rows][32 bytes], 16-byte halves swapped where (row >> 3) is odd
      const uint32_t c = static_cast<uint32_t>(8 * g + 4 * lk);             // inside the slice
      const uint32_t row = static_cast<uint32_t>(k) & 63u;
      const uint32_t half = ((c >> 4) & 1u) ^ ((row >> 3) & 1u);
      const uint32_t slices = static_cast<uint32_t>(a.C) >> 5;
      const uint32_t dst = ((((static_cast<uint32_t>(k) >> 6) * slices + blockIdx.x) * 9u + static_cast<uint32_t>(tap)) * 64u + row) * 32u + half * 16u + (c & 15u);
      *reinterpret_cast<uint32_t*>(a.wprep + dst) = wnew;
    }
  }
}

template <int Q>
int ws_resident() {
  static int resident_of[kDeviceSlots] = {};
  int& r = resident_of[device_slot()];
  if (r == 0) {
    auto k = wgrad_small_kernel<Q>;
    int dev = 0, cus = 0, per_cu = 0;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, kWsLdsBytes) != hipSuccess ||
        hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(k), 576, kWsLdsBytes) != hipSuccess)
      return 0;
    r = cus * per_cu;
  }
  return r;
}

}  // namespace

// Shapes of the one-launch form (a host-side test, no device query): any batch size - a last stage that reaches past
// the tensor reads zeros.  Sync words are those of the finishing kernel (never fewer slots).
bool wgrad_small_shape(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (R != 3 || S != 3 || stride != 1 || pad != 1 || H != W || (H != 2 && H != 4)) return false;
  if (N <= 0 || C % 32 != 0 || K % 32 != 0) return false;
  const long long pix = static_cast<long long>(N) * H * H;
  if (pix * C >= 0x7fffffffLL || pix * K >= 0x7fffffffLL || static_cast<long long>(K) * 9 * C >= 0x7fffffffLL) return false;
  const long long nb = static_cast<long long>(C / 32) * (K / 32);
  if (nb > wgrad3x3_finish_blocks(C, K)) return false;   // the caller's sync words are sized for the finishing kernel
  return pix <= 8192;                                     // long pixel ranges belong to the kernels that split them
}

// ... and whether this device holds all its workgroups at once
bool wgrad_small_supported(int N, int H, int C, int K, int w_channels) {
  if (w_channels != C || !wgrad_small_shape(N, H, H, C, K, 3, 3, 1, 1)) return false;
  const int resident = H == 2 ? ws_resident<2>() : ws_resident<4>();
  return static_cast<long long>(C / 32) * (K / 32) <= resident;
}

int launch_wgrad_small_update(const int8_t* act, const int8_t* err, int8_t* w, int N, int H, int C, int K, bool roundtrip,
                              uint32_t* sync, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep, hipStream_t stream) {
  WsArgs a{};
  a.act = act;
  a.err = err;
  a.w = w;
  a.g8 = g8;
  a.dw = dw;
  a.wprep = wprep;
  a.sync = sync;
  a.pixels = N * H * H;
  a.C = C;
  a.K = K;
  a.act_bytes = static_cast<long long>(a.pixels) * C;
  a.err_bytes = static_cast<long long>(a.pixels) * K;
  a.roundtrip = roundtrip ? 1 : 0;
  a.target_bits = rq.target_bits;
  a.method = rq.method;
  a.trunc = rq.trunc;
  a.bw_mode = rq.bw_mode;
  a.spin_limit = rq.spin_limit;
  a.sticky = rq.sticky;
  a.shift_out = rq.shift_out;
  a.exp_a = rq.exp_a;
  a.exp_b = rq.exp_b;
  a.exp_out = rq.exp_out;
  const dim3 grid(C / 32, K / 32);
  if (H == 2) hipLaunchKernelGGL(wgrad_small_kernel<2>, grid, dim3(576), kWsLdsBytes, stream, a);
  else hipLaunchKernelGGL(wgrad_small_kernel<4>, grid, dim3(576), kWsLdsBytes, stream, a);
  return check_launch("wgrad_small");
}

}  // namespace niti
