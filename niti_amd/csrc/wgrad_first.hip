// Weight gradient + grad_calc + weight update of the FIRST layer (3 input channels, 32 x 32 images) as one launch.
//
// The reference treats this layer on its own as well (ti_torch.py:194-233: a grouped convolution, because its tensor-core
// path wants channel counts in multiples of 16).  Here the reason is the shape of the work: 128 x 27 sums over 131 072
// pixels - a gradient of 3 456 numbers, one MFMA column block wide.  Run through the general kernel pair (the input
// padded to 16 channels, 256 workgroups of partial sums, a finishing launch) it takes two launches at their floor.
//
// One workgroup per image.  The 3 channel planes of the image sit in LDS with a border of zeros; the error map arrives
// in pieces of 8 image rows ([pixel][K], buffer_load ... lds, two buffers).  A reduction step is one image row of 32
// pixels: A = 32 output channels x 32 pixels by transposing LDS reads of the error tile, B = 32 columns (tap, channel) x
// 32 pixels, where a column's 16 pixels per lane are 16 consecutive bytes of a plane row, shifted by the tap's
// horizontal offset.  The workgroup adds its 32 K sums into one accumulation buffer with integer atomics (3 456 per
// image instead of 37 K partial sums per workgroup); the workgroup that arrives last holds the whole gradient and
// finishes alone - range, rounding, w = clip(w - g), the forward pass's filter copy - without any wait between
// workgroups.
#include "common.h"
#include "lds_asm.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kWfPitch = 48;                          // bytes per plane row: zero, 32 pixels, zeros; 20-byte reads at 0 and 16
constexpr int kWfPlane = 34 * kWfPitch;               // image rows -1 .. 32
constexpr int kWfXBytes = 3 * kWfPlane + 64;
constexpr int kWfCounter = 2;                         // sync word that counts the workgroups that are done
constexpr int kWfCols = 32;                           // accumulation buffer: [K][32] words, column = tap * Cw + c

struct WfArgs {
  const int8_t* act;   // [N][32][32][16], channels >= Cw are padding
  const int8_t* err;   // [N][32][32][K]
  int8_t* w;           // [K][9][Cw], updated in place
  int8_t* g8;          // optional rounded gradient, laid out like w
  int32_t* dw;         // optional int32 gradient [K][9][16]
  int8_t* wprep;       // optional kernel-ready forward filter copy (16-channel layout)
  uint32_t* sync;      // word 0 range out, word kWfCounter arrivals
  int32_t* accum;      // [K][32] zeroed words
  int N, K, Cw;
  long long err_bytes;
  int roundtrip, target_bits, method, trunc, bw_mode;
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};

template <int N>
__device__ inline void wf_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | 0x0F70);
}
__device__ inline void wf_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// KB = K / 32 blocks of output channels; the 8 wavefronts are KB blocks x (8 / KB) groups of image rows
template <int KB>
__global__ __launch_bounds__(512) void wgrad_first_kernel(const WfArgs a) {
  constexpr int K = KB * 32;
  constexpr int G = 8 / KB;              // row groups
  constexpr int RW = KB;                 // image rows per wavefront and piece of 8 rows
  constexpr int PP = K / 16;             // 16-byte pieces per pixel of the error tile
  constexpr int SWZ = PP >= 8 ? 7 : PP - 1;
  constexpr int PPI = 1024 / K;          // pixels per staging instruction
  constexpr int NBUF = K <= 128 ? 4 : 2;                   // error tiles of 8 rows in LDS
  constexpr int BUF = 256 * K;                             // the wavefronts' sums are parked across them at the end (32 KB)
  static_assert(NBUF * BUF >= 32768, "room for the parked sums");
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const planes = smem;
  int8_t* const ebuf = smem + kWfXBytes;
  __shared__ uint32_t wmax[8];
  __shared__ uint32_t flag;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kb = wave % KB, pg = wave / KB;
  const int n = blockIdx.x;

  // the image's pixels (the first dword of each holds the channels), requested ahead of the error tiles
  uint32_t xv[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) xv[h] = *reinterpret_cast<const uint32_t*>(a.act + (static_cast<long long>(n) * 1024 + tid + 512 * h) * 16);

  // The weights this lane would update if its workgroup turns out to be the last one: requested now by every workgroup
  // (3 456 bytes each), so that the finishing part does not start with a trip to memory for them.  Nobody writes them
  // before all workgroups have reported in.
  constexpr int PER = (K * 27 + 511) / 512;
  int wold[PER];
  {
    const int total_w = K * 9 * a.Cw;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = i * 512 + tid;
      wold[i] = idx < total_w ? static_cast<int>(a.w[idx]) : 0;
    }
  }

  // ---- error tile staging: an instruction fills PPI pixels x K bytes; pieces swizzled by the pixel (bank spread)
  const __amdgpu_buffer_rsrc_t rerr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.err), 0, a.err_bytes, 0x00020000);
  auto issue = [&](int piece8, int buf) {
#pragma unroll
    for (int i = 0; i < KB; ++i) {
      const int q = wave + 8 * i;                         // instruction of this piece: pixels q * PPI ..
      const int pix = q * PPI + lane / PP;
      const int slot = lane % PP;
      const int off = ((n * 1024 + piece8 * 256 + pix) * K) + ((slot ^ ((pix >> 1) & SWZ)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rerr, NITI_LDS(ebuf + buf * BUF + q * 1024), 16, off, 0, 0, 0);
    }
  };

  // ---- fragment addressing
  const int j = lane & 15, gg = (lane >> 4) & 1, lk = lane >> 5;
  unsigned a_off[2];
#pragma unroll
  for (int o = 0; o < 2; ++o) {
    const int lpix = 16 * lk + 8 * o + (j >> 1);           // inside an image row
    const int cb = kb * 32 + gg * 16 + 8 * (j & 1);
    a_off[o] = static_cast<unsigned>(lpix * K + ((((cb >> 4) ^ ((lpix >> 1) & SWZ)) << 4) | (cb & 15)));
  }
  const int col = lane & 31;                               // column (tap, channel) of the B operand
  const int ncols = 9 * a.Cw;
  const bool live = col < ncols;
  const int tap = live ? col / a.Cw : 0, ch = live ? col - tap * a.Cw : 0;
  const int dy = tap / 3, dx = tap - 3 * dy;               // 0 .. 2: plane row = image row + dy, byte shift dx
  const unsigned b_off = static_cast<unsigned>(ch * kWfPlane + dy * kWfPitch + 16 * lk);
  const unsigned lds0 = lds_addr(smem);

  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  // all four pieces of the image are requested at once where they fit (one memory latency instead of four)
  if (NBUF == 4) {
#pragma unroll
    for (int q = 0; q < 4; ++q) issue(q, q);
  } else {
    issue(0, 0);
  }
  // ---- the image's channel planes with a border of zeros, while the error tiles are on their way
  for (int i = tid; i < kWfXBytes / 4; i += 512) reinterpret_cast<uint32_t*>(planes)[i] = 0u;
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int pix = tid + 512 * h;
    const int at = ((pix >> 5) + 1) * kWfPitch + (pix & 31) + 1;
#pragma unroll
    for (int c = 0; c < 3; ++c)
      if (c < a.Cw) planes[c * kWfPlane + at] = static_cast<int8_t>((xv[h] >> (8 * c)) & 0xFFu);
  }
  static_for<4>([&](auto piecec) {
    constexpr int piece8 = decltype(piecec)::value;
    if (NBUF == 4) wf_wait_vmcnt<(3 - piece8) * KB>();     // this piece has landed (loads complete in order)
    else wf_wait_vmcnt<0>();
    wf_sync();                                             // ... for every wavefront, and the other buffer has been read
    if (NBUF != 4 && piece8 + 1 < 4) issue(piece8 + 1, (piece8 + 1) & 1);
    const unsigned ebase = lds0 + static_cast<unsigned>(kWfXBytes + (piece8 % NBUF) * BUF);
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      const int r = pg * RW + i;                           // image row inside the piece
      const unsigned ea = ebase + static_cast<unsigned>(r * 32 * K);
      const v2i alo = lds_read_tr8<0>(ea + a_off[0]);
      const v2i ahi = lds_read_tr8<0>(ea + a_off[1]);
      const unsigned ba = lds0 + b_off + static_cast<unsigned>((piece8 * 8 + r) * kWfPitch);
      const v4i d = lds_read_b128(ba);
      int d4;
      asm volatile("ds_read_b32 %0, %1 offset:16" : "=v"(d4) : "v"(ba));
      lds_settle<0>();
      const v4i fa = lds_landed(alo, ahi);
      v4i dd = d;
      asm volatile("" : "+v"(dd), "+v"(d4));
      v4i fb;
      fb[0] = static_cast<int>(__builtin_amdgcn_alignbyte(dd[1], dd[0], dx));
      fb[1] = static_cast<int>(__builtin_amdgcn_alignbyte(dd[2], dd[1], dx));
      fb[2] = static_cast<int>(__builtin_amdgcn_alignbyte(dd[3], dd[2], dx));
      fb[3] = static_cast<int>(__builtin_amdgcn_alignbyte(d4, dd[3], dx));
      if (!live) fb = v4i{0, 0, 0, 0};
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
    }
  });
  // ---- add the row groups through LDS, then into the accumulation buffer.  acc[4 g + e]: output channel
  // kb * 32 + 8 g + 4 lk + e, column lane % 32
  __syncthreads();   // every wavefront is done with the error tiles
  int* const park = reinterpret_cast<int*>(ebuf);
  if (pg > 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) park[(wave * 16 + e) * 64 + lane] = acc[e];
  }
  __syncthreads();
  if (pg == 0 && live) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      int s = acc[e];
#pragma unroll
      for (int q = 1; q < G; ++q) s += park[((q * KB + kb) * 16 + e) * 64 + lane];
      const int k = kb * 32 + 8 * (e >> 2) + 4 * lk + (e & 3);
      if (s != 0) __hip_atomic_fetch_add(a.accum + k * kWfCols + col, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // this lane's additions have been performed
  __syncthreads();
  if (tid == 0) {
    const uint32_t seen = __hip_atomic_fetch_add(a.sync + kWfCounter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    flag = seen + 1u == gridDim.x ? 1u : 0u;
  }
  __syncthreads();
  if (flag == 0u) return;

  // ---- the last workgroup holds the whole gradient: range, rounding, update
  int s[PER];
  uint32_t lmax = 0;
  const int total = K * ncols;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = i * 512 + tid;
    int v = 0;
    if (idx < total) {
      const int k = idx / ncols, c = idx - k * ncols;
      v = __hip_atomic_load(a.accum + k * kWfCols + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (a.roundtrip) v = f32_roundtrip(v);
    }
    s[i] = v;
    const uint32_t u = uabs(v);
    lmax = u > lmax ? u : lmax;
  }
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  uint32_t gmax = 0;
#pragma unroll
  for (int w8 = 0; w8 < 8; ++w8) gmax = max(gmax, wmax[w8]);
  const int shift = max(bitwidth_of(gmax, a.bw_mode) - a.target_bits, 0);
  if (tid == 0) {
    a.sync[0] = gmax;
    if (a.shift_out != nullptr) *a.shift_out = shift;
    if (a.exp_out != nullptr) *a.exp_out = shift + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
  }
  const bool trunc = a.trunc != 0, psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = i * 512 + tid;
    if (idx >= total) continue;
    const int k = idx / ncols, c9 = idx - k * ncols;
    const int t9 = c9 / a.Cw, c = c9 - t9 * a.Cw;
    int r;
    if (shift >= 1) r = psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(s[i], shift, trunc) : round_one32<NITI_ROUND_NEAREST>(s[i], shift, trunc);
    else r = wrap_to_i8(s[i]);
    const int wn = clip127(wold[i] - r);   // w is [K][9][Cw]: element idx
    a.w[idx] = static_cast<int8_t>(wn);
    if (a.g8 != nullptr) a.g8[idx] = static_cast<int8_t>(r);
    if (a.wprep != nullptr) {
      // [64-channel group][one 32-channel slice][tap][64 rows][32 bytes], 16-byte halves swapped where (row >> 3) is odd
      const uint32_t row = static_cast<uint32_t>(k) & 63u;
      const uint32_t dst = ((((static_cast<uint32_t>(k) >> 6) * 9u + static_cast<uint32_t>(t9)) * 64u + row) << 5) + ((row >> 3) & 1u) * 16u + static_cast<uint32_t>(c);
      a.wprep[dst] = static_cast<int8_t>(wn);
    }
  }
  if (a.dw != nullptr) {
    for (int idx = tid; idx < K * 9 * 16; idx += 512) {
      const int c = idx & 15, kt = idx >> 4;               // kt = k * 9 + tap
      int v = 0;
      if (c < a.Cw) {
        const int k = kt / 9, t9 = kt - 9 * k;
        v = __hip_atomic_load(a.accum + k * kWfCols + t9 * a.Cw + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (a.roundtrip) v = f32_roundtrip(v);
      }
      a.dw[idx] = v;
    }
  }
}

template <int KB>
int wf_launch(const WfArgs& a, hipStream_t stream) {
  constexpr int K = KB * 32;
  constexpr size_t lds = static_cast<size_t>(kWfXBytes) + static_cast<size_t>(K <= 128 ? 4 : 2) * 256 * K;
  auto k = wgrad_first_kernel<KB>;
  static bool attr_set_of[kDeviceSlots] = {};   // function attributes are per device
  bool& attr_set = attr_set_of[device_slot()];
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "wgrad_first: cannot reserve %zu bytes of LDS", lds);
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3(static_cast<unsigned>(a.N)), dim3(512), lds, stream, a);
  return check_launch("wgrad_first");
}

}  // namespace

// zeroed sync words the first-layer kernel wants behind the finishing kernel's (its accumulation buffer), 0 = not this shape
size_t wgrad_first_extra_words(int H, int C, int K) {
  if (H != 32 || C != 16) return 0;
  if (K != 32 && K != 64 && K != 128 && K != 256) return 0;
  return static_cast<size_t>(K) * kWfCols;
}

bool wgrad_first_supported(int N, int H, int C, int K, int w_channels) {
  if (wgrad_first_extra_words(H, C, K) == 0 || w_channels < 1 || w_channels > 3) return false;
  return static_cast<long long>(N) * 1024 * K < 0x7fffffffLL;
}

int launch_wgrad_first_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int K, bool roundtrip,
                              uint32_t* sync, int32_t* accum, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep,
                              hipStream_t stream) {
  WfArgs a{};
  a.act = act;
  a.err = err;
  a.w = w;
  a.g8 = g8;
  a.dw = dw;
  a.wprep = wprep;
  a.sync = sync;
  a.accum = accum;
  a.N = N;
  a.K = K;
  a.Cw = w_channels;
  a.err_bytes = static_cast<long long>(N) * 1024 * K;
  a.roundtrip = roundtrip ? 1 : 0;
  a.target_bits = rq.target_bits;
  a.method = rq.method;
  a.trunc = rq.trunc;
  a.bw_mode = rq.bw_mode;
  a.shift_out = rq.shift_out;
  a.exp_a = rq.exp_a;
  a.exp_b = rq.exp_b;
  a.exp_out = rq.exp_out;
  if (K == 32) return wf_launch<1>(a, stream);
  if (K == 64) return wf_launch<2>(a, stream);
  if (K == 128) return wf_launch<4>(a, stream);
  return wf_launch<8>(a, stream);
}

}  // namespace niti
