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
// The classifier at the end of a network (ti_vgg.py:37-40: TiFlat, TiDropout, TiLinear; then TiLoss) takes two launches
// of the same code: the forward kernel can also apply the dropout mask to the activations it reads (drawing the mask
// itself) and, when the targets are known, evaluate the loss gradient of the logits it has just rounded (a tile's 16
// samples are complete in its workgroup); fc_head_bwd_kernel does data gradient, dropout backward, weight gradient
// and weight update for a slab of 64 input features per workgroup.
// All of them keep their int32 sums in registers across the tensor-wide range: every workgroup publishes its
// largest magnitude in a slot of its own and reads all slots (all workgroups resident - checked by the host - and
// the wait bounded by a wall-clock limit), as the convolution kernels do.
#include <stdlib.h>

#include "common.h"
#include "lds_asm.h"
#include "loss_math.h"
#include "requant_math.h"
#include "rng.h"

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
  // classifier head, forward only
  int dropout;               // 0 none, 1 mask given, 2 mask drawn from rng and written to mask
  int8_t* mask;              // [F] 0 / 1 per input feature
  uint32_t* rng;             // generator state (rng.h)
  int exp_bias;              // added to the output exponent (the dropout's + 1)
  const int64_t* target;     // [M] or null: with it the loss gradient of the rounded logits is written as well
  const int32_t* loss_rand;  // [M][O] low four bits used, or null (then drawn from rng)
  int8_t* loss_grad;         // [M][O]
};

__device__ inline int round_to_i8(int x, int shift, bool psto, bool trunc) {
  if (shift < 1) return wrap_to_i8(x);
  return psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, shift, trunc) : round_one32<NITI_ROUND_NEAREST>(x, shift, trunc);
}

__device__ inline void write_scalars(const FcArgs& a, uint32_t gmax, int shift) {
  const int sh = shift > 0 ? shift : 0;
  a.sync[0] = gmax;
  if (a.shift_out != nullptr) *a.shift_out = sh;
  if (a.exp_out != nullptr) *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0) + a.exp_bias;
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
// kHead: dropout on the activations (mask bytes 0x00 / 0xFF in dynamic LDS, F bytes) and the loss gradient.
// kLds (F and kchunk multiples of 128): the fragments do not come straight from memory - 64-byte pieces of the rows,
// which the path from L2 into a compute unit moves at a third of the rate of whole 128-byte lines, and that path is what
// bounds a workgroup that pulls 26 rows of F bytes - but every wavefront stages its share one line per row at a time
// (buffer_load ... lds: an instruction moves eight rows' lines, lane -> (row lane / 8, 16-byte piece lane % 8), pieces
// XOR-swizzled by the row, every instruction's kilobyte 16 bytes further on, so that the fragment reads spread over the
// banks) in two buffers of its own: no barrier in the loop, the next line on its way while this one multiplies.
constexpr int kFsInstrBytes = 1024 + 16;
constexpr int kFsStage = 4 * kFsInstrBytes;            // 16 weight rows + 16 samples, one line each
constexpr int kFsStagesBytes = 16 * 2 * kFsStage;      // 16 wavefronts x 2 buffers
template <bool kHead, bool kLds = false>
__global__ __launch_bounds__(1024) void fc_fwd_requant_kernel(const FcArgs a) {
  __shared__ int part[16][256];
  __shared__ __attribute__((aligned(16))) int8_t logits[16][16];   // kHead: the tile's rounded logits
  extern __shared__ __attribute__((aligned(16))) unsigned char keep_base[];   // kLds: the stages come first, then the mask
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int mt = blockIdx.x;
  const bool drop = kHead && a.dropout != 0;
  const bool draws = kHead && (a.dropout == 2 || (a.target != nullptr && a.loss_rand == nullptr));
  unsigned char* const keep = kLds ? keep_base + kFsStagesBytes : keep_base;
  // kLds: the first line is requested before anything else, so that it travels while the mask is made
  const int k0 = wave * a.kchunk;
  [[maybe_unused]] int nlines = 0;
  [[maybe_unused]] int src[4] = {0, 0, 0, 0};
  [[maybe_unused]] unsigned stage0 = 0;
  [[maybe_unused]] const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(a.w, 0, a.O * a.F, 0x00020000);
  [[maybe_unused]] const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.act), 0, a.M * a.F, 0x00020000);
  auto issue = [&](int line, int buf) {
    const int kb = k0 + line * 128;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned dst = stage0 + buf * kFsStage + j * kFsInstrBytes;
      if (j < 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS_AT(dst), 16, src[j], kb, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, NITI_LDS_AT(dst), 16, src[j], kb, 0, 0);
    }
  };
  if constexpr (kLds) {
    nlines = k0 < a.F ? (min(k0 + a.kchunk, a.F) - k0) >> 7 : 0;
    const int r8 = lane >> 3, piece = (lane & 7) ^ r8;
#pragma unroll
    for (int j = 0; j < 4; ++j) {                      // instruction j: rows 8 j .. 8 j + 7 of the panel (16 weight rows, 16 samples)
      const int prow = 8 * j + r8;
      const int g = prow < 16 ? prow : mt * 16 + prow - 16;
      const bool in = prow < 16 ? g < a.O : g < a.M;
      src[j] = in ? g * a.F + piece * 16 : static_cast<int>(0x80000000u);   // out of range whatever scalar offset is added: zeros
    }
    stage0 = lds_addr(keep_base) + wave * (2 * kFsStage);
    if (nlines > 0) issue(0, 0);
  }
  // the sample's target class is wanted at the very end, behind a chain of waits: requested now
  long long target_of_row = -1;
  if (kHead && a.target != nullptr && wave < 4) {
    const int trow = mt * 16 + wave * 4 + (lane >> 4);
    if (trow < a.M) target_of_row = a.target[trow];
  }
  RngDraw draw{};
  if (draws) draw = rng_read(a.rng);
  if (drop) {
    for (int k = threadIdx.x * 8; k < a.F; k += 1024 * 8) {   // F is a multiple of 16
      uint32_t m[2];
      if (a.dropout == 2) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          uint32_t w4[4];
          rng_words4(draw, kRngStreamDropout, static_cast<uint32_t>(k / 4 + h), w4);
          m[h] = (w4[0] & 1u) | ((w4[1] & 1u) << 8) | ((w4[2] & 1u) << 16) | ((w4[3] & 1u) << 24);
        }
        if (mt == 0) {
          *reinterpret_cast<uint32_t*>(a.mask + k) = m[0];
          *reinterpret_cast<uint32_t*>(a.mask + k + 4) = m[1];
        }
      } else {
        m[0] = *reinterpret_cast<const uint32_t*>(a.mask + k);
        m[1] = *reinterpret_cast<const uint32_t*>(a.mask + k + 4);
      }
      *reinterpret_cast<uint32_t*>(keep + k) = m[0] * 255u;      // bytes 0 / 1 -> 0x00 / 0xFF
      *reinterpret_cast<uint32_t*>(keep + k + 4) = m[1] * 255u;
    }
    __syncthreads();
  }
  const int row = lane & 15, kg = lane >> 4;           // operand row (sample / output feature), 16-byte piece of a 64-step
  const int m = mt * 16 + row;
  const int k1 = min(k0 + a.kchunk, a.F);
  const int8_t* pa = a.act + static_cast<long long>(m) * a.F;
  const int8_t* pw = a.w + static_cast<long long>(row) * a.F;
  const bool va = m < a.M, vw = row < a.O;
  v4i acc = {0, 0, 0, 0};
  const v4i zero = {0, 0, 0, 0};
  if constexpr (kLds) {
    // fragments: lane (row, kg) of 64-step s reads piece 4 s + kg of its row's line
    const unsigned frow = (row >> 3) * kFsInstrBytes + (row & 7) * 128;
    unsigned fpiece[2];
#pragma unroll
    for (int sstep = 0; sstep < 2; ++sstep) fpiece[sstep] = static_cast<unsigned>(((4 * sstep + kg) ^ (row & 7)) * 16);
    const unsigned keep0 = lds_addr(keep) + k0 + kg * 16;
    for (int line = 0; line < nlines; ++line) {
      const int buf = line & 1;
      if (line + 1 < nlines) {
        issue(line + 1, buf ^ 1);
        __builtin_amdgcn_s_waitcnt(0x0F70 | 4);                      // vmcnt(4): this line has landed, the next one is on its way
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                          // vmcnt(0)
      }
      const unsigned base = stage0 + buf * kFsStage + frow;
      v4i fw[2], fa[2], fk[2];
#pragma unroll
      for (int sstep = 0; sstep < 2; ++sstep) {
        fw[sstep] = lds_read_b128(base + fpiece[sstep]);
        fa[sstep] = lds_read_b128(base + 2 * kFsInstrBytes + fpiece[sstep]);
        if (drop) fk[sstep] = lds_read_b128(keep0 + line * 128 + sstep * 64);
      }
      lds_settle<0>();
#pragma unroll
      for (int sstep = 0; sstep < 2; ++sstep) {
        asm volatile("" : "+v"(fw[sstep]), "+v"(fa[sstep]));
        if (drop) {
          asm volatile("" : "+v"(fk[sstep]));
          fa[sstep] &= fk[sstep];
        }
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[sstep], fw[sstep], acc, 0, 0, 0);
      }
    }
  } else
  for (int kb = k0; kb < k1; kb += 256) {                 // four 64-steps at a time, their loads in flight together
    v4i fa[4], fw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = kb + u * 64 + kg * 16;
      const bool in = k < k1;                             // F is a multiple of 16: a piece is inside or outside
      fa[u] = (va && in) ? *reinterpret_cast<const v4i*>(pa + k) : zero;
      fw[u] = (vw && in) ? *reinterpret_cast<const v4i*>(pw + k) : zero;
      if (drop && in) fa[u] &= *reinterpret_cast<const v4i*>(keep + k);
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
      int r = 0;
      if (mm < a.M && o < a.O) {
        r = round_to_i8(acc[i], shift, psto, trunc);
        if (relu && r < 0) r = 0;
        a.out8[static_cast<long long>(mm) * a.O + o] = static_cast<int8_t>(r);
      }
      if (kHead) logits[4 * (lane >> 4) + i][o] = static_cast<int8_t>(r);
    }
    if (kHead && lane == 0) part[0][0] = (shift > 0 ? shift : 0) + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0) + a.exp_bias;
  }
  if (!kHead) return;
  if (a.target != nullptr) {
    // ti_loss.py:5-36 for the tile's samples: sixteen lanes per sample (one per class), four samples per wavefront
    __syncthreads();
    if (wave < 4) {
      const int e = part[0][0];
      const int srow = wave * 4 + (lane >> 4), j = lane & 15;
      const int row = mt * 16 + srow;
      const bool valid = row < a.M && j < a.O;
      const int v = logits[srow][j];
      const bool big = e > -7, up = e >= 0;
      const float p2 = exp2f(static_cast<float>(up ? e : -e));   // exact power of two
      auto group_sum = [](long long x) {
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
          const int lo = __shfl_xor(static_cast<int>(x & 0xFFFFFFFFLL), off, 64);
          const int hi = __shfl_xor(static_cast<int>(x >> 32), off, 64);
          x += (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo);
        }
        return x;
      };
      float nm;             // out_grad before the normalisation, as float32
      long long term;       // its truncation (ti_loss.py:31)
      if (big) {
        const float sc = scaled_logit(v, p2, up);
        float mx = valid ? sc : -INFINITY;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        nm = exp2_contract(fmaxf(sc - (mx - 10.0f), 0.0f)) - 1.0f;
        term = static_cast<long long>(nm);
      } else {
        term = loss_small_term(v, e);
        nm = static_cast<float>(term);
      }
      const float fsum = static_cast<float>(group_sum(valid ? term : 0LL));
      float g = nm * 2048.0f / fsum;
      const long long tsum = group_sum(valid ? static_cast<long long>(g) : 0LL);   // ti_loss.py:34
      if (valid) {
        if (j == target_of_row) g = g - static_cast<float>(tsum);
        const int x = static_cast<int>(g);   // .type(torch.int32)
        const long long idx = static_cast<long long>(row) * a.O + j;
        const int u = a.loss_rand != nullptr ? a.loss_rand[idx] & 15 : static_cast<int>(rng_word(draw, kRngStreamLoss, static_cast<uint32_t>(idx)) & 15u);
        a.loss_grad[idx] = static_cast<int8_t>(round_one<NITI_ROUND_STOCHASTIC>(x, 4, a.trunc != 0, u));
      }
    }
  }
  if (draws && threadIdx.x == 0) rng_arrive(a.rng, gridDim.x, draw);
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

// ---- classifier head, backward: data gradient + dropout backward + weight gradient + update -----------------------
// ti_torch.py:255-266 followed by ti_torch.py:452-455 in one launch.  A workgroup owns a slab of 64 input features:
// it stages the error rows (all samples, 16 bytes each), the slab of the weights as stored and the slab of the
// activations with the dropout mask applied (what the forward pass multiplied), then
//   dx[m][f] = sum_o err[m][o] w[o][f]   sixteen wavefronts x 16 samples, four MFMAs each,
//   g[o][f]  = sum_m err[m][o] act[m][f] four wavefronts x 16 features, an MFMA per 64 samples,
// (v_mfma_i32_16x16x64_i8; weights and activations are transposed on their way into LDS),
// exchanges both ranges, rounds, masks and stores dx, and applies w = clip(w - g) to its slab.
constexpr int kHeadSlab = 64;
constexpr int kHeadMaxM = 256;     // a lane holds four samples x 16 features of the data gradient

struct HeadBwdArgs {
  const int8_t* err;    // [M][O]
  const int8_t* act;    // [M][F], before the dropout
  const int8_t* mask;   // [F] 0 / 1, or null
  int8_t* w;            // [O][F], updated in place
  int8_t* dx8;          // [M][F]
  int8_t* g8;           // [O][F] rounded gradient, or null
  uint32_t* sync;       // 0 data-gradient range, 1 wait gave up, 2 weight-gradient range, kSlot0.. a slot of two words per workgroup
  int M, O, F;
  int err_bits, err_method, grad_bits, grad_method, trunc, bw_mode;
  long long spin_limit;
  uint32_t* sticky;
  int32_t* err_shift_out;
  int32_t* grad_shift_out;
  const int32_t* exp_err;
  const int32_t* exp_w;
  const int32_t* exp_act;
  int exp_act_bias;
  int32_t* err_exp_out;
  int32_t* grad_exp_out;
  // backward pass of the 2 x 2 max-pool whose flattened output act is ([M][P][Q][C], F = P Q C, C a multiple of 64)
  const int8_t* pool_in;   // [M][2P][2Q][C], or null
  int8_t* unpooled;        // [M][2P][2Q][C]
  int pool_q, pool_c;
  int pool_ties_all, pool_relu;
};

__device__ inline int byte_of(uint32_t w, int b) { return static_cast<int>(static_cast<int8_t>((w >> (8 * b)) & 0xFFu)); }

// 4 x 4 byte transposition: in[j] holds bytes 0..3 of row j; out[b] holds byte b of rows 0..3
__device__ inline void transpose4x4_bytes(const uint32_t (&in)[4], uint32_t (&out)[4]) {
  const uint32_t lo01 = __builtin_amdgcn_perm(in[1], in[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(in[1], in[0], 0x07030602u);
  const uint32_t lo23 = __builtin_amdgcn_perm(in[3], in[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(in[3], in[2], 0x07030602u);
  out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
  out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
  out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
  out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

constexpr int kHeadGroups = kHeadMaxM / 4;     // groups of four samples
constexpr int kHeadActPitch = kHeadGroups + 4; // words per feature row of the transposed activations (16-byte rows, banks spread)

// wait_slots for slots that hold two values: workgroup b stores (data-gradient maximum + 1) | (weight-gradient
// maximum + 1) << 32 as one 8-byte word at slot b.  Called by a whole wavefront; nb <= 4096.
static_assert(kSlotStride % 2 == 0, "a slot must hold an 8-byte aligned pair of words");
__device__ inline void wait_slot_pairs(uint32_t* slots, int nb, long long spin_limit, uint32_t* timed_out, uint32_t* sticky,
                                       uint32_t& max_lo, uint32_t& max_hi) {
  const int lane = threadIdx.x & 63;
  const long long t0 = wall_clock64();
  uint32_t glo = 0, ghi = 0;
  bool gave_up = false;
  for (int base = 0; base < nb && !gave_up; base += 64) {
    unsigned long long v = base + lane < nb ? 0ULL : 1ULL;
    for (;;) {
      if (v == 0ULL)
        v = __hip_atomic_load(reinterpret_cast<unsigned long long*>(slot_word(slots, base + lane)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__all(v != 0ULL) && spin_limit > 0) break;
      if (spin_limit <= 0 || wall_clock64() - t0 > spin_limit) {   // a limit of zero: give up after the first look (tests)
        if (lane == 0) {
          __hip_atomic_fetch_or(timed_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (sticky != nullptr) __hip_atomic_store(sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(4);
    }
    if (base + lane < nb) {
      const uint32_t lo = static_cast<uint32_t>(v), hi = static_cast<uint32_t>(v >> 32);
      glo = lo > glo ? lo : glo;
      ghi = hi > ghi ? hi : ghi;
    }
  }
  max_lo = wave_max_u32(glo);
  max_hi = wave_max_u32(ghi);
}

__global__ __launch_bounds__(1024, 8) void fc_head_bwd_kernel(const HeadBwdArgs a) {
  // both products run on v_mfma_i32_16x16x64_i8, whose operands are rows with the reduction index in consecutive bytes
  __shared__ __attribute__((aligned(16))) uint32_t err_s[kHeadMaxM * 4];               // [m][o]: 16 bytes per sample
  __shared__ __attribute__((aligned(16))) uint32_t err_t[kMaxOut * kHeadGroups];       // [o][m]
  __shared__ __attribute__((aligned(16))) uint32_t act_t[kHeadSlab * kHeadActPitch];   // [f][m], masked
  __shared__ __attribute__((aligned(16))) uint32_t w_t[kHeadSlab * 4];                 // [f][o]: 16 bytes per input feature
  __shared__ __attribute__((aligned(16))) uint32_t keep_s[kHeadSlab / 4];              // dropout mask of the slab as 0x00 / 0xFF bytes
  __shared__ uint32_t wmax_d[16], wmax_w[16], gshare[2];
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int f0 = blockIdx.x * kHeadSlab;
  const v4i zero = {0, 0, 0, 0};
  if (t < 256) {
    const int piece = t & 3, mgroup = t >> 2;     // 16-byte piece of the slab, group of four samples
    v4i mk = {-1, -1, -1, -1};
    if (a.mask != nullptr) {
      const v4i m = *reinterpret_cast<const v4i*>(a.mask + f0 + piece * 16);
#pragma unroll
      for (int d = 0; d < 4; ++d) mk[d] = static_cast<int>(static_cast<uint32_t>(m[d]) * 255u);   // bytes 0 / 1 -> 0x00 / 0xFF
    }
    v4i av[4];      // samples 4 mgroup .. + 3, features f0 + 16 piece .. + 15
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = 4 * mgroup + j;
      av[j] = m < a.M ? *reinterpret_cast<const v4i*>(a.act + static_cast<long long>(m) * a.F + f0 + piece * 16) : zero;
    }
    uint32_t win[4] = {0u, 0u, 0u, 0u};
    if (t < 64) {   // weights: output features 4 (t / 16) .. + 3, input features f0 + 4 (t % 16) .. + 3
#pragma unroll
      for (int j = 0; j < 4; ++j)
        win[j] = 4 * (t >> 4) + j < a.O ? *reinterpret_cast<const uint32_t*>(a.w + static_cast<long long>(4 * (t >> 4) + j) * a.F + f0 + 4 * (t & 15)) : 0u;
    }
    uint32_t eb[kMaxOut];   // error row of sample t, all loads in flight together
#pragma unroll
    for (int o = 0; o < kMaxOut; ++o)
      eb[o] = (t < a.M && o < a.O) ? static_cast<uint32_t>(a.err[static_cast<long long>(t) * a.O + o]) & 0xFFu : 0u;
    if (t < 4) *reinterpret_cast<v4i*>(keep_s + 4 * t) = mk;
    if (t < 64) {
      uint32_t out[4];
      transpose4x4_bytes(win, out);
#pragma unroll
      for (int b = 0; b < 4; ++b) w_t[(4 * (t & 15) + b) * 4 + (t >> 4)] = out[b];
    }
    uint32_t wd[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int o = 0; o < kMaxOut; ++o) wd[o >> 2] |= eb[o] << (8 * (o & 3));
    *reinterpret_cast<v4i*>(err_s + t * 4) = v4i{static_cast<int>(wd[0]), static_cast<int>(wd[1]), static_cast<int>(wd[2]), static_cast<int>(wd[3])};
#pragma unroll
    for (int d = 0; d < 4; ++d) {   // activations, masked, transposed: word d of the four rows -> features 4 d .. 4 d + 3
      const uint32_t in[4] = {static_cast<uint32_t>(av[0][d] & mk[d]), static_cast<uint32_t>(av[1][d] & mk[d]),
                              static_cast<uint32_t>(av[2][d] & mk[d]), static_cast<uint32_t>(av[3][d] & mk[d])};
      uint32_t out[4];
      transpose4x4_bytes(in, out);
#pragma unroll
      for (int b = 0; b < 4; ++b) act_t[(16 * piece + 4 * d + b) * kHeadActPitch + mgroup] = out[b];
    }
  }
  __syncthreads();
  {               // err_t[o][g] from err_s: one word per thread (16 output features x 64 groups)
    const int o = t >> 6, g = t & 63;
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) word |= ((err_s[(4 * g + j) * 4 + (o >> 2)] >> (8 * (o & 3))) & 0xFFu) << (8 * j);
    err_t[o * kHeadGroups + g] = word;
  }
  // data gradient: wavefront w takes samples 16 w .. + 15; per block of 16 features one MFMA whose reduction (the
  // output features) fills the first quarter of its 64 steps.  dacc[blk][i]: feature 16 blk + 4 (lane / 16) + i of
  // sample 16 w + lane % 16
  const int row = lane & 15, kg = lane >> 4;
  v4i dacc[4];
  {
    const v4i eop = kg == 0 ? *reinterpret_cast<const v4i*>(err_s + (16 * wave + row) * 4) : zero;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      const v4i wop = kg == 0 ? *reinterpret_cast<const v4i*>(w_t + (16 * blk + row) * 4) : zero;
      dacc[blk] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop, eop, zero, 0, 0, 0);
    }
  }
  __syncthreads();   // err_t is complete
  // weight gradient: wavefront w < 4 takes features 16 w .. + 15, 64 samples per MFMA.  gacc[i]: output feature
  // 4 (lane / 16) + i, feature 16 w + lane % 16
  v4i gacc = zero;
  if (wave < 4) {
    const int steps = (a.M + 63) >> 6;
    for (int ks = 0; ks < steps; ++ks) {
      const v4i eop = *reinterpret_cast<const v4i*>(err_t + row * kHeadGroups + ks * 16 + kg * 4);
      const v4i aop = *reinterpret_cast<const v4i*>(act_t + (16 * wave + row) * kHeadActPitch + ks * 16 + kg * 4);
      gacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(eop, aop, gacc, 0, 0, 0);
    }
  }
  uint32_t dmax = 0, gmaxl = 0;
#pragma unroll
  for (int blk = 0; blk < 4; ++blk)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t u = uabs(dacc[blk][i]);     // rows beyond M are sums of zeros
      dmax = u > dmax ? u : dmax;
    }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t u = uabs(gacc[i]);
    gmaxl = u > gmaxl ? u : gmaxl;
  }
  dmax = wave_max_u32(dmax);
  gmaxl = wave_max_u32(gmaxl);
  if (lane == 0) {
    wmax_d[wave] = dmax;
    wmax_w[wave] = gmaxl;
  }
  __syncthreads();
  if (wave == 0) {
    const uint32_t bd = wave_max_u32(lane < 16 ? wmax_d[lane] : 0u);
    const uint32_t bw = wave_max_u32(lane < 16 ? wmax_w[lane] : 0u);
    uint32_t* const slots = a.sync + kSlot0;
    if (lane == 0)
      __hip_atomic_store(reinterpret_cast<unsigned long long*>(slot_word(slots, blockIdx.x)),
                         static_cast<unsigned long long>(bd + 1u) | (static_cast<unsigned long long>(bw + 1u) << 32), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    uint32_t gd = 0, gw = 0;
    wait_slot_pairs(slots, gridDim.x, a.spin_limit, &a.sync[1], a.sticky, gd, gw);
    if (lane == 0) {
      gshare[0] = gd != 0u ? gd - 1u : 0u;
      gshare[1] = gw != 0u ? gw - 1u : 0u;
    }
  }
  __syncthreads();
  const uint32_t range_d = gshare[0], range_w = gshare[1];
  const int shift_d = bitwidth_of(range_d, a.bw_mode) - a.err_bits;
  const int shift_w = bitwidth_of(range_w, a.bw_mode) - a.grad_bits;
  if (blockIdx.x == 0 && t == 0) {
    const int sd = shift_d > 0 ? shift_d : 0, sw = shift_w > 0 ? shift_w : 0;
    a.sync[0] = range_d;
    a.sync[2] = range_w;
    const int e_err = sd + (a.exp_err != nullptr ? *a.exp_err : 0) + (a.exp_w != nullptr ? *a.exp_w : 0);   // ti_torch.py:260
    if (a.err_shift_out != nullptr) *a.err_shift_out = sd;
    if (a.grad_shift_out != nullptr) *a.grad_shift_out = sw;
    if (a.err_exp_out != nullptr) *a.err_exp_out = e_err;
    if (a.grad_exp_out != nullptr) *a.grad_exp_out = sw + e_err + (a.exp_act != nullptr ? *a.exp_act : 0) + a.exp_act_bias;   // ti_torch.py:18
  }
  // the pool window of this thread's (sample, 16 channels) is requested here, ahead of the rounding and the stores of the
  // two gradients (any earlier and the kernel needs more registers than let two workgroups share a compute unit)
  const bool unpool = a.pool_in != nullptr && t < a.M * 4;
  long long px0 = 0, prowb = 0;
  v4i py = zero, px[4] = {zero, zero, zero, zero};
  if (unpool) {
    const int m = t >> 2, piece = t & 3;
    const int pp = f0 / a.pool_c, c = f0 - pp * a.pool_c + piece * 16;
    const int ph = pp / a.pool_q, pw = pp - ph * a.pool_q;
    prowb = static_cast<long long>(2 * a.pool_q) * a.pool_c;
    px0 = ((static_cast<long long>(m) * 2 * (a.F / (a.pool_q * a.pool_c)) + 2 * ph) * 2 * a.pool_q + 2 * pw) * a.pool_c + c;
    py = *reinterpret_cast<const v4i*>(a.act + static_cast<long long>(m) * a.F + f0 + piece * 16);
    px[0] = *reinterpret_cast<const v4i*>(a.pool_in + px0);
    px[1] = *reinterpret_cast<const v4i*>(a.pool_in + px0 + a.pool_c);
  }
  const bool trunc = a.trunc != 0;
  const bool psto_d = a.err_method == NITI_ROUND_PSEUDO_STOCHASTIC, psto_w = a.grad_method == NITI_ROUND_PSEUDO_STOCHASTIC;
  {
    const int m = 16 * wave + row;
    if (m < a.M) {
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        const uint32_t r4 = pack4_i8(round_to_i8(dacc[blk][0], shift_d, psto_d, trunc), round_to_i8(dacc[blk][1], shift_d, psto_d, trunc),
                                     round_to_i8(dacc[blk][2], shift_d, psto_d, trunc), round_to_i8(dacc[blk][3], shift_d, psto_d, trunc));
        const uint32_t kept = r4 & keep_s[4 * blk + kg];   // ti_torch.py:454
        if (a.dx8 != nullptr) *reinterpret_cast<uint32_t*>(a.dx8 + static_cast<long long>(m) * a.F + f0 + 16 * blk + 4 * kg) = kept;
        if (a.pool_in != nullptr) act_t[m * (kHeadSlab / 4) + 4 * blk + kg] = kept;   // [m][64 bytes]: the transposed activations are done with
      }
    }
  }
  if (wave < 4) {
    const int f = 16 * wave + row;
    const uint32_t wold = w_t[f * 4 + kg];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int o = 4 * kg + i;
      if (o < a.O) {
        const int r = round_to_i8(gacc[i], shift_w, psto_w, trunc);
        const long long at = static_cast<long long>(o) * a.F + f0 + f;
        a.w[at] = static_cast<int8_t>(clip127(byte_of(wold, i) - r));
        if (a.g8 != nullptr) a.g8[at] = static_cast<int8_t>(r);
      }
    }
  }
  if (a.pool_in == nullptr) return;
  // ---- the max-pool's backward pass for the slab (64 channels of one pooled pixel): thread (sample, 16 channels)
  // routes its 16 gradients to the window positions that hold the maximum (int8pool_kernel.cu:84-138; the first in scan
  // order, or all of them), zeroed where the pool's input is not positive when the ReLU in front leaves that to it
  __syncthreads();
  if (unpool) {
    const int m = t >> 2, piece = t & 3;
    const long long x0 = px0, rowb = prowb;
    const v4i y = py;
    const v4i d = *reinterpret_cast<const v4i*>(act_t + m * (kHeadSlab / 4) + piece * 4);
    px[2] = *reinterpret_cast<const v4i*>(a.pool_in + px0 + prowb);   // the window's second row: requested late, for want of registers
    px[3] = *reinterpret_cast<const v4i*>(a.pool_in + px0 + prowb + a.pool_c);
    const v4i (&x)[4] = px;
    v4i o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint32_t taken = 0;   // bytes whose gradient an earlier position of the window (scan order) already received
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t eq = equal_bytes(static_cast<uint32_t>(x[k][e]), static_cast<uint32_t>(y[e]));
        uint32_t keep = a.pool_ties_all ? eq : eq & ~taken;
        if (a.pool_relu) keep &= positive_bytes(static_cast<uint32_t>(x[k][e]));
        o[k][e] = static_cast<int>(static_cast<uint32_t>(d[e]) & keep);
        taken |= eq;
      }
    }
    *reinterpret_cast<v4i*>(a.unpooled + x0) = o[0];
    *reinterpret_cast<v4i*>(a.unpooled + x0 + a.pool_c) = o[1];
    *reinterpret_cast<v4i*>(a.unpooled + x0 + rowb) = o[2];
    *reinterpret_cast<v4i*>(a.unpooled + x0 + rowb + a.pool_c) = o[3];
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

// The forward kernel's LDS-staged form: taken when F is a multiple of 128, its stages (and the dropout mask) fit beside
// the kernel's static LDS and one workgroup per compute unit covers the grid.  NITI_FC_LDS=0 pins the other form.
template <bool kHead>
bool fwd_lds_ok(int F, long long nb, size_t mask_bytes, size_t* lds) {
  *lds = static_cast<size_t>(kFsStagesBytes) + mask_bytes;
  const char* e = getenv("NITI_FC_LDS");
  if ((e != nullptr && e[0] == '0') || F % 128 != 0 || *lds + 16384 + 256 + 64 > 160 * 1024) return false;
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) {
    // counted with the largest allocation the kernel takes, so the answer holds for every call
    constexpr int kMost = 160 * 1024 - 16384 - 256 - 64;
    int dev = 0, cus = 0, per_cu = 0;
    const void* k = reinterpret_cast<const void*>(fc_fwd_requant_kernel<kHead, true>);
    if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kMost) == hipSuccess && hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k, 1024, kMost) == hipSuccess)
      resident = cus * per_cu;
    if (resident == 0) resident = -1;
  }
  return nb <= resident;
}

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
  if (resident == 0) resident = resident_blocks(reinterpret_cast<const void*>(fc_fwd_requant_kernel<false>), 1024);
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "fc_fwd_requant: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  a.kchunk = fwd_chunk(F);
  size_t lds_staged = 0;
  if (fwd_lds_ok<false>(F, nb, 0, &lds_staged))
    hipLaunchKernelGGL((fc_fwd_requant_kernel<false, true>), dim3(static_cast<unsigned>(nb)), dim3(1024), lds_staged, static_cast<hipStream_t>(stream), a);
  else
    hipLaunchKernelGGL((fc_fwd_requant_kernel<false, false>), dim3(static_cast<unsigned>(nb)), dim3(1024), 0, static_cast<hipStream_t>(stream), a);
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

// ---- classifier head ------------------------------------------------------------------------------------------
static long long head_bwd_blocks(int M, int O, int F) {
  if (M <= 0 || O <= 0 || F <= 0 || O > kMaxOut || M > kHeadMaxM || F % kHeadSlab != 0) return 0;
  const long long nb = F / kHeadSlab;
  return nb <= 4096 ? nb : 0;
}

extern "C" size_t niti_head_i8_sync_words(int backward, int M, int O, int F) {
  if (!backward) return niti_fc_i8_sync_words(NITI_FC_FORWARD, M, O, F);
  const long long nb = head_bwd_blocks(M, O, F);
  if (nb == 0) return 0;
  return static_cast<size_t>(kSlot0) + slot_words(static_cast<int>(nb));
}

extern "C" int niti_head_i8_forward(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int dropout,
                                    int8_t* drop_mask, uint32_t* rng, int exp_bias, const int64_t* target, const int32_t* loss_rand,
                                    int8_t* loss_grad, int target_bits, int method, int div_mode, int bw_mode, unsigned rq_flags,
                                    uint32_t* sync, size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                    int32_t* exp_out, void* stream) {
  FcArgs a{};
  long long nb = 0;
  const int st = fc_common("head_forward", NITI_FC_FORWARD, a, M, O, F, target_bits, method, div_mode, bw_mode, sync, sync_words,
                           shift_out, exp_a, exp_b, exp_out, &nb);
  if (st != NITI_OK) return st;
  if (act == nullptr || w == nullptr || out8 == nullptr) return fail(NITI_ERR_INVALID_ARG, "head_forward: null pointer");
  if (!aligned16(act) || !aligned16(w)) return fail(NITI_ERR_INVALID_ARG, "head_forward: operands must be 16-byte aligned");
  if (dropout < 0 || dropout > 2) return fail(NITI_ERR_INVALID_ARG, "head_forward: dropout=%d (0 none, 1 mask given, 2 mask drawn)", dropout);
  if (dropout != 0 && (drop_mask == nullptr || reinterpret_cast<uintptr_t>(drop_mask) % 4 != 0))
    return fail(NITI_ERR_INVALID_ARG, "head_forward: the dropout mask must be a 4-byte aligned array of F bytes");
  if (dropout != 0 && F > 32768) return fail(NITI_ERR_UNSUPPORTED, "head_forward: dropout over more than 32768 features");
  if (target != nullptr && loss_grad == nullptr) return fail(NITI_ERR_INVALID_ARG, "head_forward: targets without a place for the loss gradient");
  if ((dropout == 2 || (target != nullptr && loss_rand == nullptr)) && rng == nullptr)
    return fail(NITI_ERR_INVALID_ARG, "head_forward: random draws asked for without a generator state");
  if (static_cast<long long>(M) * O > 0x7FFFFFFFLL) return fail(NITI_ERR_UNSUPPORTED, "head_forward: more than 2^31 logits");
  a.act = act;
  a.w = const_cast<int8_t*>(w);
  a.out8 = out8;
  a.rq_flags = rq_flags;
  a.dropout = dropout;
  a.mask = drop_mask;
  a.rng = rng;
  a.exp_bias = exp_bias;
  a.target = target;
  a.loss_rand = loss_rand;
  a.loss_grad = loss_grad;
  const size_t lds = dropout != 0 ? static_cast<size_t>(F) : 0;
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) {
    // counted with the largest mask the kernel takes, so the answer holds for every call
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(fc_fwd_requant_kernel<true>), 1024, 32768) == hipSuccess)
      resident = cus * per_cu;
  }
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "head_forward: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  a.kchunk = fwd_chunk(F);
  size_t lds_staged = 0;
  if (fwd_lds_ok<true>(F, nb, lds, &lds_staged))
    hipLaunchKernelGGL((fc_fwd_requant_kernel<true, true>), dim3(static_cast<unsigned>(nb)), dim3(1024), lds_staged, static_cast<hipStream_t>(stream), a);
  else
    hipLaunchKernelGGL((fc_fwd_requant_kernel<true, false>), dim3(static_cast<unsigned>(nb)), dim3(1024), lds, static_cast<hipStream_t>(stream), a);
  return check_launch("head_forward");
}

static int head_backward(const int8_t* err, const int8_t* act, const int8_t* drop_mask, int8_t* w, int8_t* dx8, int M, int O,
                         int F, int err_bits, int err_method, int grad_bits, int grad_method, int div_mode, int bw_mode,
                         uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* err_shift_out, int32_t* grad_shift_out,
                         const int32_t* exp_err, const int32_t* exp_w, const int32_t* exp_act, int exp_act_bias,
                         int32_t* err_exp_out, int32_t* grad_exp_out, const int8_t* pool_in, int8_t* unpooled, int P, int Q, int C,
                         int pool_flags, void* stream) {
  clear_error();
  if (M <= 0 || O <= 0 || F <= 0) return fail(NITI_ERR_INVALID_ARG, "head_backward: non-positive extent");
  if (err == nullptr || act == nullptr || w == nullptr || sync == nullptr || (dx8 == nullptr && pool_in == nullptr))
    return fail(NITI_ERR_INVALID_ARG, "head_backward: null pointer");
  int ties = 0;
  if (pool_in != nullptr) {
    ties = pool_flags & ~NITI_POOL_BWD_RELU;
    if (ties != NITI_TIES_FIRST && ties != NITI_TIES_ALL) return fail(NITI_ERR_INVALID_ARG, "head_backward_unpool: ties=%d", ties);
    if (unpooled == nullptr || !aligned16(pool_in) || !aligned16(unpooled))
      return fail(NITI_ERR_INVALID_ARG, "head_backward_unpool: the pool's input and the result must be 16-byte aligned arrays");
    if (P <= 0 || Q <= 0 || C <= 0 || C % kHeadSlab != 0 || static_cast<long long>(P) * Q * C != F)
      return fail(NITI_ERR_UNSUPPORTED, "head_backward_unpool: F=%d is not P=%d x Q=%d x C=%d with C a multiple of %d", F, P, Q, C, kHeadSlab);
    if (4LL * M * F >= 0x7fffffffLL) return fail(NITI_ERR_UNSUPPORTED, "head_backward_unpool: more than 2^31 elements");
  }
  if (err_bits < 1 || err_bits > 7 || grad_bits < 1 || grad_bits > 7)
    return fail(NITI_ERR_INVALID_ARG, "head_backward: err_bits=%d grad_bits=%d outside 1..7", err_bits, grad_bits);
  for (const int method : {err_method, grad_method})
    if (method != NITI_ROUND_NEAREST && method != NITI_ROUND_PSEUDO_STOCHASTIC)
      return fail(NITI_ERR_UNSUPPORTED, "head_backward: rounding method %d needs random input; use the separate passes", method);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "head_backward: div_mode=%d", div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "head_backward: bw_mode=%d", bw_mode);
  const long long nb = head_bwd_blocks(M, O, F);
  if (nb == 0)
    return fail(NITI_ERR_UNSUPPORTED, "head_backward: M=%d O=%d F=%d outside the kernel (M <= %d, O <= %d, F a multiple of %d); use the separate passes",
                M, O, F, kHeadMaxM, kMaxOut, kHeadSlab);
  if (!aligned16(act) || !aligned16(w) || (dx8 != nullptr && !aligned16(dx8)) || (drop_mask != nullptr && !aligned16(drop_mask)))
    return fail(NITI_ERR_INVALID_ARG, "head_backward: act, w, dx8 and the mask must be 16-byte aligned");
  const size_t need = niti_head_i8_sync_words(1, M, O, F);
  if (sync_words < need) return fail(NITI_ERR_WORKSPACE, "head_backward: needs %zu zeroed sync words, got %zu", need, sync_words);
  static int resident_of[kDeviceSlots] = {};
  int& resident = resident_of[device_slot()];
  if (resident == 0) resident = resident_blocks(reinterpret_cast<const void*>(fc_head_bwd_kernel), 1024);
  if (nb > resident) return fail(NITI_ERR_UNSUPPORTED, "head_backward: %lld workgroups do not fit on the device at once (%d)", nb, resident);
  HeadBwdArgs a{};
  a.err = err;
  a.act = act;
  a.mask = drop_mask;
  a.w = w;
  a.dx8 = dx8;
  a.g8 = g8_out;
  a.sync = sync;
  a.M = M;
  a.O = O;
  a.F = F;
  a.err_bits = err_bits;
  a.err_method = err_method;
  a.grad_bits = grad_bits;
  a.grad_method = grad_method;
  a.trunc = div_mode == NITI_DIV_TRUNC ? 1 : 0;
  a.bw_mode = bw_mode;
  a.spin_limit = sync_spin_limit();
  a.sticky = timeout_word();
  a.err_shift_out = err_shift_out;
  a.grad_shift_out = grad_shift_out;
  a.exp_err = exp_err;
  a.exp_w = exp_w;
  a.exp_act = exp_act;
  a.exp_act_bias = exp_act_bias;
  a.err_exp_out = err_exp_out;
  a.grad_exp_out = grad_exp_out;
  a.pool_in = pool_in;
  a.unpooled = unpooled;
  a.pool_q = Q;
  a.pool_c = C;
  a.pool_ties_all = ties == NITI_TIES_ALL ? 1 : 0;
  a.pool_relu = (pool_flags & NITI_POOL_BWD_RELU) != 0 ? 1 : 0;
  hipLaunchKernelGGL(fc_head_bwd_kernel, dim3(static_cast<unsigned>(nb)), dim3(1024), 0, static_cast<hipStream_t>(stream), a);
  return check_launch("head_backward");
}

extern "C" int niti_head_i8_backward(const int8_t* err, const int8_t* act, const int8_t* drop_mask, int8_t* w, int8_t* dx8, int M, int O,
                                     int F, int err_bits, int err_method, int grad_bits, int grad_method, int div_mode, int bw_mode,
                                     uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* err_shift_out, int32_t* grad_shift_out,
                                     const int32_t* exp_err, const int32_t* exp_w, const int32_t* exp_act, int exp_act_bias,
                                     int32_t* err_exp_out, int32_t* grad_exp_out, void* stream) {
  if (dx8 == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "head_backward: null pointer");
  }
  return head_backward(err, act, drop_mask, w, dx8, M, O, F, err_bits, err_method, grad_bits, grad_method, div_mode, bw_mode, sync, sync_words,
                       g8_out, err_shift_out, grad_shift_out, exp_err, exp_w, exp_act, exp_act_bias, err_exp_out, grad_exp_out, nullptr, nullptr,
                       0, 0, 0, 0, stream);
}

extern "C" int niti_head_i8_backward_unpool(const int8_t* err, const int8_t* act, const int8_t* drop_mask, int8_t* w, int8_t* dx8, int M,
                                            int O, int F, int err_bits, int err_method, int grad_bits, int grad_method, int div_mode,
                                            int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* err_shift_out,
                                            int32_t* grad_shift_out, const int32_t* exp_err, const int32_t* exp_w, const int32_t* exp_act,
                                            int exp_act_bias, int32_t* err_exp_out, int32_t* grad_exp_out, const int8_t* pool_in,
                                            int8_t* unpooled, int P, int Q, int C, int pool_flags, void* stream) {
  if (pool_in == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "head_backward_unpool: null pointer");
  }
  return head_backward(err, act, drop_mask, w, dx8, M, O, F, err_bits, err_method, grad_bits, grad_method, div_mode, bw_mode, sync, sync_words,
                       g8_out, err_shift_out, grad_shift_out, exp_err, exp_w, exp_act, exp_act_bias, err_exp_out, grad_exp_out, pool_in, unpooled,
                       P, Q, C, pool_flags, stream);
}
