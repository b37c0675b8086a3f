// TiLinear with few output features (the classifier: 8192 -> 10), each direction as one launch with its
// requantisation folded in (ti_torch.py:241-266).  A GEMM with a 10-wide dimension leaves the tiled MFMA
// kernels one ragged tile and two operand re-layouts; written for the shape, all three passes read their
// operands as stored:
//   forward   out[m][o] = sum_f act[m][f] w[o][f]   -> act_calc: both operands are reduction-contiguous, which is
//             the register layout of v_mfma_i32_16x16x64_i8; a workgroup owns 16 samples, its 16 wavefronts split
//             the reduction and are added through LDS.
//   dgrad     dx[m][f] = sum_o err[m][o] w[o][f]    -> err_calc: a lane owns 16 consecutive f of one sample.
//   wgrad     g[o][f]  = sum_m err[m][o] act[m][f]  -> grad_calc -> w = clip(w - g): a lane owns 4 consecutive f,
//             the four wavefronts of a workgroup each take a quarter of the samples (four at a time through
//             v_dot4_i32_i8 after a 4 x 4 byte transposition) and are added through LDS.
// All three keep their int32 sums in registers across the tensor-wide range: every workgroup publishes its
// largest magnitude in a slot of its own and reads all slots (all workgroups resident - checked by the host - and
// the wait bounded by a wall-clock limit), as the convolution kernels do.
#include "common.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kSlot0 = 16;      // sync words: 0 range out, 1 wait gave up, 16.. one slot per workgroup
constexpr int kMaxOut = 16;     // output features these kernels handle
constexpr int kWgradMaxM = 512;

struct FcArgs {
  const int8_t* act;   // [M][F]
  const int8_t* err;   // [M][O]
  int8_t* w;           // [O][F] (read only except in the weight update)
  int8_t* out8;        // forward: [M][O]; dgrad: [M][F]; wgrad: optional rounded gradient [O][F]
  uint32_t* sync;
  int M, O, F;
  int kchunk;          // forward: reduction elements per wavefront
  int target_bits, method, trunc, bw_mode;
  unsigned rq_flags;
  long long spin_limit;
  uint32_t* sticky;   // device-wide word set when the wait gives up, may be null
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};

__device__ inline int round_to_i8(int x, int shift, bool psto, bool trunc) {
  if (shift < 1) return wrap_to_i8(x);
  return psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, shift, trunc) : round_one32<NITI_ROUND_NEAREST>(x, shift, trunc);
}

__device__ inline void write_scalars(const FcArgs& a, uint32_t gmax, int shift) {
  const int sh = shift > 0 ? shift : 0;
  a.sync[0] = gmax;
  if (a.shift_out != nullptr) *a.shift_out = sh;
  if (a.exp_out != nullptr) *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
}

// Called by wavefront 0 of every workgroup with the workgroup's largest magnitude: returns the largest over the grid.
__device__ inline uint32_t exchange_range(const FcArgs& a, uint32_t bmax) {
  const int lane = threadIdx.x & 63;
  const int nb = gridDim.x;
  uint32_t* const slots = a.sync + kSlot0;
  if (lane == 0) __hip_atomic_store(slot_word(slots, blockIdx.x), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint32_t g = wait_slots(slots, nb, a.spin_limit, &a.sync[1], a.sticky);
  return g != 0u ? g - 1u : 0u;
}

// ---- forward ------------------------------------------------------------------------------------------
// One workgroup of 16 wavefronts per tile of 16 samples; wavefront w reduces over features [w * kchunk, (w+1) * kchunk).
__global__ __launch_bounds__(1024) void fc_fwd_requant_kernel(const FcArgs a) {
  __shared__ int part[16][256];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int mt = blockIdx.x;
  const int row = lane & 15, kg = lane >> 4;           // operand row (sample / output feature), 16-byte piece of a 64-step
  const int m = mt * 16 + row;
  const int k0 = wave * a.kchunk;
  const int k1 = min(k0 + a.kchunk, a.F);
  const int8_t* pa = a.act + static_cast<long long>(m) * a.F;
  const int8_t* pw = a.w + static_cast<long long>(row) * a.F;
  const bool va = m < a.M, vw = row < a.O;
  v4i acc = {0, 0, 0, 0};
  const v4i zero = {0, 0, 0, 0};
  for (int kb = k0; kb < k1; kb += 256) {                 // four 64-steps at a time, their loads in flight together
    v4i fa[4], fw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = kb + u * 64 + kg * 16;
      const bool in = k < k1;                             // F is a multiple of 16: a piece is inside or outside
      fa[u] = (va && in) ? *reinterpret_cast<const v4i*>(pa + k) : zero;
      fw[u] = (vw && in) ? *reinterpret_cast<const v4i*>(pw + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[u], fw[u], acc, 0, 0, 0);
  }
  // acc[i]: sample mt*16 + 4*(lane/16) + i, output feature lane%16
#pragma unroll
  for (int i = 0; i < 4; ++i) part[wave][i * 64 + lane] = acc[i];
  __syncthreads();
  if (wave == 0) {
    uint32_t lmax = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < 16; ++w) sum += part[w][i * 64 + lane];
      acc[i] = sum;
      const uint32_t u = uabs(sum);     // rows beyond M and columns beyond O are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
    const uint32_t gmax = exchange_range(a, wave_max_u32(lmax));
    const int shift = bitwidth_of(gmax, a.bw_mode) - a.target_bits;
    if (blockIdx.x == 0 && lane == 0) write_scalars(a, gmax, shift);
    const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC, trunc = a.trunc != 0, relu = (a.rq_flags & NITI_RQ_RELU) != 0;
    const int o = lane & 15;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int mm = mt * 16 + 4 * (lane >> 4) + i;
      if (mm < a.M && o < a.O) {
        int r = round_to_i8(acc[i], shift, psto, trunc);
        if (relu && r < 0) r = 0;
        a.out8[static_cast<long long>(mm) * a.O + o] = static_cast<int8_t>(r);
      }
    }
  }
}

// ---- data gradient ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fc_dgrad_requant_kernel(const FcArgs a) {
  __shared__ uint32_t wmax[4];
  __shared__ uint32_t gshare;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fv = a.F >> 4;
  const long long t = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  const bool valid = t < static_cast<long long>(a.M) * fv;
  const int m = valid ? static_cast<int>(t / fv) : 0;
  const int f = valid ? static_cast<int>(t - static_cast<long long>(m) * fv) * 16 : 0;
  int acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0;
  {
    // all rows of w at once (rows beyond O repeat the last one with a zero factor): sixteen loads in flight
    v4i wv[kMaxOut];
    int e[kMaxOut];
#pragma unroll
    for (int o = 0; o < kMaxOut; ++o) {
      const int oo = min(o, a.O - 1);
      wv[o] = *reinterpret_cast<const v4i*>(a.w + static_cast<long long>(oo) * a.F + f);
      e[o] = (valid && o < a.O) ? static_cast<int>(a.err[static_cast<long long>(m) * a.O + oo]) : 0;
    }
#pragma unroll
    for (int o = 0; o < kMaxOut; ++o)
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[4 * d + b] += e[o] * static_cast<int>(static_cast<int8_t>((static_cast<uint32_t>(wv[o][d]) >> (8 * b)) & 0xFFu));
  }
  uint32_t lmax = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t u = uabs(acc[i]);
    lmax = u > lmax ? u : lmax;
  }
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  if (wave == 0) {
    uint32_t b = wmax[0];
    b = max(max(b, wmax[1]), max(wmax[2], wmax[3]));
    const uint32_t g = exchange_range(a, b);
    if (lane == 0) gshare = g;
  }
  __syncthreads();
  const uint32_t gmax = gshare;
  const int shift = bitwidth_of(gmax, a.bw_mode) - a.target_bits;
  if (blockIdx.x == 0 && threadIdx.x == 0) write_scalars(a, gmax, shift);
  if (!valid) return;
  const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC, trunc = a.trunc != 0;
  v4i o4;
#pragma unroll
  for (int d = 0; d < 4; ++d)
    o4[d] = static_cast<int>(pack4_i8(round_to_i8(acc[4 * d], shift, psto, trunc), round_to_i8(acc[4 * d + 1], shift, psto, trunc),
                                      round_to_i8(acc[4 * d + 2], shift, psto, trunc), round_to_i8(acc[4 * d + 3], shift, psto, trunc)));
  *reinterpret_cast<v4i*>(a.out8 + static_cast<long long>(m) * a.F + f) = o4;
}

// ---- weight gradient + update ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fc_wgrad_update_kernel(const FcArgs a) {
  // one buffer used twice: the error words during the loop, the four wavefronts' sums after it
  __shared__ __attribute__((aligned(16))) int smem_raw[4 * kMaxOut * 4 * 64];
  __shared__ uint32_t wmax[4];
  __shared__ uint32_t gshare;
  static_assert(sizeof(uint32_t) * kMaxOut * (kWgradMaxM / 4) <= sizeof(smem_raw), "error words fit the buffer");
  uint32_t (*err_t)[kWgradMaxM / 4] = reinterpret_cast<uint32_t (*)[kWgradMaxM / 4]>(smem_raw);   // [o][sample / 4]
  int (*red)[kMaxOut * 4][64] = reinterpret_cast<int (*)[kMaxOut * 4][64]>(smem_raw);              // [wavefront][o * 4 + b][lane]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int groups = (a.M + 3) >> 2;                      // groups of four samples
  const int f = (blockIdx.x * 64 + lane) * 4;
  const bool valid = f < a.F;                              // F is a multiple of 4
  const int per = (groups + 3) >> 2;
  const int g0 = wave * per, g1 = min(g0 + per, groups);
  const int8_t* pa = a.act + f;
  constexpr int kAhead = 4;   // groups of four samples whose loads are in flight together
  auto load = [&](int gb, uint32_t (&r)[kAhead][4]) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = 4 * (gb + u) + j;
        r[u][j] = (valid && gb + u < g1 && m < a.M) ? *reinterpret_cast<const uint32_t*>(pa + static_cast<long long>(m) * a.F) : 0u;
      }
  };
  uint32_t ra[kAhead][4], rb[kAhead][4];
  load(g0, ra);                                             // in flight while the error words are put together
  for (int i = threadIdx.x; i < kMaxOut * groups; i += 256) {
    const int o = i / groups, g = i - o * groups;
    uint32_t word = 0;
    if (o < a.O) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = 4 * g + j;
        if (m < a.M) word |= (static_cast<uint32_t>(a.err[static_cast<long long>(m) * a.O + o]) & 0xFFu) << (8 * j);
      }
    }
    err_t[o][g] = word;
  }
  __syncthreads();
  int acc[kMaxOut][4];
#pragma unroll
  for (int o = 0; o < kMaxOut; ++o)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[o][b] = 0;
  auto mac = [&](int gb, const uint32_t (&r)[kAhead][4]) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const int g = min(gb + u, groups - 1);   // beyond g1 the loaded activations are zero
      // 4 x 4 byte transposition: c[b] = byte b (feature f + b) of the four samples
      const uint32_t lo01 = __builtin_amdgcn_perm(r[u][1], r[u][0], 0x05010400u), hi01 = __builtin_amdgcn_perm(r[u][1], r[u][0], 0x07030602u);
      const uint32_t lo23 = __builtin_amdgcn_perm(r[u][3], r[u][2], 0x05010400u), hi23 = __builtin_amdgcn_perm(r[u][3], r[u][2], 0x07030602u);
      uint32_t c[4];
      c[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
      c[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
      c[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
      c[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
#pragma unroll
      for (int o = 0; o < kMaxOut; ++o) {
        if (o < a.O) {
          const int ew = static_cast<int>(err_t[o][g]);
#pragma unroll
          for (int b = 0; b < 4; ++b) acc[o][b] = __builtin_amdgcn_sdot4(static_cast<int>(c[b]), ew, acc[o][b], false);
        }
      }
    }
  };
  for (int gb = g0; gb < g1; gb += 2 * kAhead) {
    load(gb + kAhead, rb);
    mac(gb, ra);
    load(gb + 2 * kAhead, ra);
    mac(gb + kAhead, rb);
  }
  __syncthreads();   // every wavefront is done with the error words
#pragma unroll
  for (int o = 0; o < kMaxOut; ++o)
#pragma unroll
    for (int b = 0; b < 4; ++b) red[wave][o * 4 + b][lane] = acc[o][b];
  __syncthreads();
  // wavefront w completes, rounds and applies the output features w, w + 4, w + 8, w + 12
  int fin[4][4];
  uint32_t lmax = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int row = (4 * j + wave) * 4 + b;
      fin[j][b] = red[0][row][lane] + red[1][row][lane] + red[2][row][lane] + red[3][row][lane];
      const uint32_t u = uabs(fin[j][b]);
      lmax = u > lmax ? u : lmax;
    }
  uint32_t wcur[4];   // the weights this lane updates, fetched while the ranges are exchanged
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = 4 * j + wave;
    wcur[j] = (valid && o < a.O) ? *reinterpret_cast<const uint32_t*>(a.w + static_cast<long long>(o) * a.F + f) : 0u;
  }
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  if (wave == 0) {
    const uint32_t g = exchange_range(a, max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
    if (lane == 0) gshare = g;
  }
  __syncthreads();
  const uint32_t gmax = gshare;
  const int shift = bitwidth_of(gmax, a.bw_mode) - a.target_bits;
  if (blockIdx.x == 0 && threadIdx.x == 0) write_scalars(a, gmax, shift);
  if (!valid) return;
  const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC, trunc = a.trunc != 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = 4 * j + wave;
    if (o < a.O) {
      const uint32_t wold = wcur[j];
      int r[4];
      uint32_t wnew = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        r[b] = round_to_i8(fin[j][b], shift, psto, trunc);
        const int wo = static_cast<int>(static_cast<int8_t>((wold >> (8 * b)) & 0xFFu));
        wnew |= (static_cast<uint32_t>(clip127(wo - r[b])) & 0xFFu) << (8 * b);
      }
      *reinterpret_cast<uint32_t*>(a.w + static_cast<long long>(o) * a.F + f) = wnew;
      if (a.out8 != nullptr) *reinterpret_cast<uint32_t*>(a.out8 + static_cast<long long>(o) * a.F + f) = pack4_i8(r[0], r[1], r[2], r[3]);
    }
  }
}

int resident_blocks(const void* kernel, int threads = 256) {
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess)
    return 0;
  return cus * per_cu;
}

// forward: reduction elements per wavefront (a multiple of 256), sixteen wavefronts per 16-sample tile
int fwd_chunk(int F) { return ((F + 15) / 16 + 255) / 256 * 256; }

long long blocks_of(int which, int M, int O, int F) {
  if (M <= 0 || O <= 0 || F <= 0 || O > kMaxOut) return 0;
  if (which == NITI_FC_FORWARD) {
    if (F % 16 != 0) return 0;
    const long long nb = (M + 15) / 16;
    return nb <= 4096 ? nb : 0;
  }
  if (which == NITI_FC_DGRAD) {
    if (F % 16 != 0) return 0;
    const long long nb = (static_cast<long long>(M) * (F / 16) + 255) / 256;
    return nb <= 4096 ? nb : 0;
  }
  if (which == NITI_FC_WGRAD) {
    if (F % 4 != 0 || M > kWgradMaxM) return 0;
    const long long nb = (F / 4 + 63) / 64;
    return nb <= 4096 ? nb : 0;
  }
  return 0;
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" size_t niti_fc_i8_sync_words(int which, int M, int O, int F) {
  const long long nb = blocks_of(which, M, O, F);
  if (nb == 0) return 0;
  return static_cast<size_t>(kSlot0) + slot_words(static_cast<int>(nb));
}

static int fc_common(const char* who, int which, FcArgs& a, int M, int O, int F, int target_bits, int method, int div_mode,
                     int bw_mode, uint32_t* sync, size_t sync_words, int32_t* shift_out, const int32_t* exp_a,
                     const int32_t* exp_b, int32_t* exp_out, long long* blocks) {
  clear_error();
  if (M <= 0 || O <= 0 || F <= 0) return fail(NITI_ERR_INVALID_ARG, "%s: non-positive extent", who);
  if (sync == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (target_bits < 1 || target_bits > 7) return fail(NITI_ERR_INVALID_ARG, "%s: target_bits=%d outside 1..7", who, target_bits);
  if (method != NITI_ROUND_NEAREST && method != NITI_ROUND_PSEUDO_STOCHASTIC)
    return fail(NITI_ERR_UNSUPPORTED, "%s: rounding method %d needs random input; use the GEMM and requantisation entry points", who, method);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "%s: div_mode=%d", who, div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "%s: bw_mode=%d", who, bw_mode);
  *blocks = blocks_of(which, M, O, F);
  if (*blocks == 0) return fail(NITI_ERR_UNSUPPORTED, "%s: M=%d O=%d F=%d outside the few-output-features kernels; use the GEMM entry point", who, M, O, F);
  const size_t need = niti_fc_i8_sync_words(which, M, O, F);
  if (sync_words < need) return fail(NITI_ERR_WORKSPACE, "%s: needs %zu zeroed sync words, got %zu", who, need, sync_words);
  a.sync = sync;
  a.M = M;
  a.O = O;
  a.F = F;
  a.target_bits = target_bits;
  a.method = method;
  a.trunc = div_mode == NITI_DIV_TRUNC ? 1 : 0;
  a.bw_mode = bw_mode;
  a.spin_limit = sync_spin_limit();
  a.sticky = timeout_word();
  a.shift_out = shift_out;
  a.exp_a = exp_a;
  a.exp_b = exp_b;
  a.exp_out = exp_out;
  return NITI_OK;
}

extern "C" int niti_fc_i8_fwd_requant(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int target_bits,
                                      int method, int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words,
                                      int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                      void* stream) {
  FcArgs a{};
  long long nb = 0;
  const int st = fc_common("fc_fwd_requant", NITI_FC_FORWARD, a, M, O, F, target_bits, method, div_mode, bw_mode, sync, sync_words,
                           shift_out, exp_a, exp_b, exp_out, &nb);
  if (st != NITI_OK) return st;
  if (act == nullptr || w == nullptr || out8 == nullptr) return fail(NITI_ERR_INVALID_ARG, "fc_fwd_requant: null pointer");
  if (!aligned16(act) || !aligned16(w)) return fail(NITI_ERR_INVALID_ARG, "fc_fwd_requant: operands must be 16-byte aligned");
  a.act = act;
  a.w = const_cast<int8_t*>(w);
  a.out8 = out8;
  a.rq_flags = rq_flags;
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) resident = resident_blocks(reinterpret_cast<const void*>(fc_fwd_requant_kernel), 1024);
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "fc_fwd_requant: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  a.kchunk = fwd_chunk(F);
  hipLaunchKernelGGL(fc_fwd_requant_kernel, dim3(static_cast<unsigned>(nb)), dim3(1024), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("fc_fwd_requant");
}

extern "C" int niti_fc_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int M, int O, int F, int target_bits,
                                        int method, int div_mode, int bw_mode, uint32_t* sync, size_t sync_words,
                                        int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                        void* stream) {
  FcArgs a{};
  long long nb = 0;
  const int st = fc_common("fc_dgrad_requant", NITI_FC_DGRAD, a, M, O, F, target_bits, method, div_mode, bw_mode, sync, sync_words,
                           shift_out, exp_a, exp_b, exp_out, &nb);
  if (st != NITI_OK) return st;
  if (err == nullptr || w == nullptr || dx8 == nullptr) return fail(NITI_ERR_INVALID_ARG, "fc_dgrad_requant: null pointer");
  if (!aligned16(w) || !aligned16(dx8)) return fail(NITI_ERR_INVALID_ARG, "fc_dgrad_requant: w and dx8 must be 16-byte aligned");
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) resident = resident_blocks(reinterpret_cast<const void*>(fc_dgrad_requant_kernel));
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "fc_dgrad_requant: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  a.err = err;
  a.w = const_cast<int8_t*>(w);
  a.out8 = dx8;
  hipLaunchKernelGGL(fc_dgrad_requant_kernel, dim3(static_cast<unsigned>(nb)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("fc_dgrad_requant");
}

extern "C" int niti_fc_i8_wgrad_update(const int8_t* err, const int8_t* act, int8_t* w, int M, int O, int F, int mu, int method,
                                       int div_mode, int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out,
                                       int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                       void* stream) {
  FcArgs a{};
  long long nb = 0;
  const int st = fc_common("fc_wgrad_update", NITI_FC_WGRAD, a, M, O, F, mu, method, div_mode, bw_mode, sync, sync_words, shift_out,
                           exp_a, exp_b, exp_out, &nb);
  if (st != NITI_OK) return st;
  if (err == nullptr || act == nullptr || w == nullptr) return fail(NITI_ERR_INVALID_ARG, "fc_wgrad_update: null pointer");
  if (reinterpret_cast<uintptr_t>(act) % 4 != 0 || reinterpret_cast<uintptr_t>(w) % 4 != 0 || reinterpret_cast<uintptr_t>(g8_out) % 4 != 0)
    return fail(NITI_ERR_INVALID_ARG, "fc_wgrad_update: act, w and g8_out must be 4-byte aligned");
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) resident = resident_blocks(reinterpret_cast<const void*>(fc_wgrad_update_kernel));
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "fc_wgrad_update: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  a.err = err;
  a.act = act;
  a.w = w;
  a.out8 = g8_out;
  hipLaunchKernelGGL(fc_wgrad_update_kernel, dim3(static_cast<unsigned>(nb)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("fc_wgrad_update");
}
