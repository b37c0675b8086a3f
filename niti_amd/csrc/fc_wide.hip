// TiLinear of any width (ti_torch.py:241-266), each pass as one launch on the matrix cores with its requantisation
// folded in - including stochastic rounding on random integers the caller supplies.  All three passes read their
// operands as the layer stores them (act [M][F], w [O][F], err [M][O]); the reference transposes and copies three
// times per step (ti_torch.py:246,263,176) and writes every int32 product to memory before rounding it.
//
//   forward   out[m][o] = sum_f act[m][f] w[o][f]: both operands are reduction-contiguous, i.e. they already are MFMA
//             fragments (v_mfma_i32_16x16x64_i8, 16 bytes per lane straight from memory).  A workgroup owns 16 output
//             features x MT x 16 samples; its 16 wavefronts split the reduction and are added through LDS.
//   dgrad     dx[m][f] = sum_o err[m][o] w[o][f]: the reduction index is the slow one of w.  A workgroup owns 32
//             features: it stages w[:, f0 .. f0+32) as stored (O rows of 32 bytes) and reads the operand fragments
//             with ds_read_b64_tr_b8, which hands each lane eight consecutive rows of one byte column; the error rows
//             are reduction-contiguous and come straight from memory.  8 wavefronts = 4 tiles of 32 samples x 2 halves
//             of the reduction.
//   wgrad     g[o][f] = sum_m err[m][o] act[m][f] -> grad_calc -> w = clip(w - g): the reduction index (samples) is the
//             slow one of both operands, both are staged as stored and transposed by the LDS read.  A workgroup owns 256
//             features x T x 32 output features; the products leave the MFMA layout through LDS so that every lane
//             updates 16 consecutive weights of one row.
// The int32 sums stay in registers across the tensor-wide range: every workgroup publishes its largest magnitude in a
// slot of its own and reads all slots (all workgroups resident - checked by the host - wait bounded by a wall clock).
#include <stdlib.h>

#include "common.h"
#include "lds_asm.h"
#include "nn_lines.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kSlot0 = 16;   // sync words: 0 range out, 1 wait gave up, 16.. one slot per workgroup

struct FcwArgs {
  const int8_t* act;     // [M][F]
  const int8_t* err;     // [M][O]
  int8_t* w;             // [O][F] (written only by the weight update)
  int8_t* out8;          // forward [M][O]; dgrad [M][F]; wgrad: optional rounded gradient [O][F]
  const int32_t* rand;   // one per output element, NITI_ROUND_STOCHASTIC only
  uint32_t* sync;
  int M, O, F;
  int kchunk;            // forward: reduction elements per wavefront
  int target_bits, method, trunc, bw_mode;
  unsigned rq_flags;
  long long spin_limit;
  uint32_t* sticky;
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};

__device__ inline int round_any(int x, int shift, int method, bool trunc, int u) {
  if (shift < 1) return wrap_to_i8(x);
  if (method == NITI_ROUND_STOCHASTIC) return round_one<NITI_ROUND_STOCHASTIC>(x, shift, trunc, u & ((1 << shift) - 1));
  return method == NITI_ROUND_PSEUDO_STOCHASTIC ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, shift, trunc)
                                                : round_one32<NITI_ROUND_NEAREST>(x, shift, trunc);
}

__device__ inline void write_scalars(const FcwArgs& a, uint32_t gmax, int shift) {
  const int sh = shift > 0 ? shift : 0;
  a.sync[0] = gmax;
  if (a.shift_out != nullptr) *a.shift_out = sh;
  if (a.exp_out != nullptr) *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
}

// Called by wavefront 0 of every workgroup with the workgroup's largest magnitude: the largest over the grid.
__device__ inline uint32_t exchange_range(const FcwArgs& a, uint32_t bmax) {
  const int lane = threadIdx.x & 63;
  const int nb = gridDim.x * gridDim.y;
  const int b = blockIdx.y * gridDim.x + blockIdx.x;
  uint32_t* const slots = a.sync + kSlot0;
  if (lane == 0) __hip_atomic_store(slot_word(slots, b), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const uint32_t g = wait_slots(slots, nb, a.spin_limit, &a.sync[1], a.sticky);
  return g != 0u ? g - 1u : 0u;
}

// the workgroup's shift from every wavefront's largest magnitude: wmax[] holds one word per wavefront, gshare the result
template <int NWAVES>
__device__ inline int grid_shift(const FcwArgs& a, uint32_t lmax, uint32_t* wmax, uint32_t* gshare) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  if (wave == 0) {
    uint32_t b = lane < NWAVES ? wmax[lane] : 0u;
    b = wave_max_u32(b);
    const uint32_t g = exchange_range(a, b);
    if (lane == 0) *gshare = g;
  }
  __syncthreads();
  const uint32_t gmax = *gshare;
  const int shift = bitwidth_of(gmax, a.bw_mode) - a.target_bits;
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) write_scalars(a, gmax, shift);
  return shift;
}

// barrier that the compiler also treats as a fence for the hand-written LDS reads around it
__device__ inline void sync_mem() {
  asm volatile("" ::: "memory");
  __syncthreads();
  asm volatile("" ::: "memory");
}

// ---- forward ------------------------------------------------------------------------------------------------
// grid.x = 16-feature tiles of the output, grid.y = groups of MT 16-sample tiles.  MFMA A = w rows (output features),
// B = act rows (samples): result element i of a lane is output feature 4 * (lane / 16) + i of sample lane % 16, i.e.
// four consecutive bytes of an output row.
template <int MT>
__global__ __launch_bounds__(1024) void fcw_fwd_kernel(const FcwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int (*part)[MT * 256] = reinterpret_cast<int (*)[MT * 256]>(smem);     // [16 wavefronts][MT tiles x 4 x 64]
  uint32_t* const words = reinterpret_cast<uint32_t*>(smem + 16 * MT * 256 * 4);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, kg = lane >> 4;
  const int o = blockIdx.x * 16 + row;
  const int m0 = blockIdx.y * (MT * 16);
  const int k0 = wave * a.kchunk;
  const int k1 = min(k0 + a.kchunk, a.F);
  const int8_t* pw = a.w + static_cast<long long>(min(o, a.O - 1)) * a.F;
  const int8_t* pa[MT];
  bool va[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = m0 + t * 16 + row;
    va[t] = m < a.M;
    pa[t] = a.act + static_cast<long long>(min(m, a.M - 1)) * a.F;
  }
  const bool vw = o < a.O;
  v4i acc[MT];
  const v4i zero = {0, 0, 0, 0};
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = zero;
  for (int kb = k0; kb < k1; kb += 256) {                 // four 64-steps at a time, their loads in flight together
    v4i fw[4], fa[MT][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = kb + u * 64 + kg * 16;
      const bool in = k < k1;                             // F is a multiple of 16: a piece is inside or outside
      fw[u] = (vw && in) ? *reinterpret_cast<const v4i*>(pw + k) : zero;
#pragma unroll
      for (int t = 0; t < MT; ++t) fa[t][u] = (va[t] && in) ? *reinterpret_cast<const v4i*>(pa[t] + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[u], fa[t][u], acc[t], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][t * 256 + i * 64 + lane] = acc[t][i];
  __syncthreads();
  // wavefront t completes tile t (wavefronts beyond MT only take part in the barriers)
  uint32_t lmax = 0;
  v4i fin = zero;
  if (wave < MT) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < 16; ++w) sum += part[w][wave * 256 + i * 64 + lane];
      fin[i] = sum;
      const uint32_t u = uabs(sum);                        // rows beyond M and columns beyond O are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
  }
  const int shift = grid_shift<16>(a, lmax, words, words + 16);
  if (wave >= MT) return;
  const int m = m0 + wave * 16 + (lane & 15);
  const int ob = blockIdx.x * 16 + 4 * (lane >> 4);
  if (m >= a.M || ob >= a.O) return;                       // O is a multiple of 4: a dword is inside or outside
  const bool trunc = a.trunc != 0, relu = (a.rq_flags & NITI_RQ_RELU) != 0;
  const long long at = static_cast<long long>(m) * a.O + ob;
  v4i u = zero;
  if (a.method == NITI_ROUND_STOCHASTIC) u = *reinterpret_cast<const v4i*>(a.rand + at);
  int r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = round_any(fin[i], shift, a.method, trunc, u[i]);
    if (relu && r[i] < 0) r[i] = 0;
  }
  *reinterpret_cast<uint32_t*>(a.out8 + at) = pack4_i8(r[0], r[1], r[2], r[3]);
}

// ---- forward, operands through LDS --------------------------------------------------------------------------
// The kernel above fetches its fragments as 64-byte pieces of the rows, which the path from L2 into a compute unit
// moves at well under half the rate of whole 128-byte lines - and that path is what bounds this pass (a workgroup
// pulls (16 + MT * 16) rows of F bytes).  Here (F a multiple of 128) every wavefront stages its share of the reduction
// one line per row at a time (buffer_load ... lds: an instruction moves eight rows' lines, lane -> (row lane / 8,
// 16-byte piece lane % 8), pieces XOR-swizzled by the row so that the fragment reads below spread over the banks; every
// instruction's kilobyte starts 16 bytes further on for the same reason) and reads the MFMA fragments from there.
// Eight wavefronts split the reduction; a wavefront only ever reads what it loaded itself, so the loop needs no
// barrier: two buffers per wavefront, the next line on its way while this one multiplies.
constexpr int kFwdInstrBytes = 1024 + 16;
template <int MT>
constexpr int fwd_lds_stage_bytes() { return (2 + 2 * MT) * kFwdInstrBytes; }
template <int MT>
__global__ __launch_bounds__(512) void fcw_fwd_lds_kernel(const FcwArgs a) {
  constexpr int NI = 2 + 2 * MT;                      // load instructions per line: 16 weight rows, MT x 16 sample rows
  constexpr int STAGE = fwd_lds_stage_bytes<MT>();
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];   // 8 wavefronts x 2 stages; later the partial sums
  int (*part)[MT * 256] = reinterpret_cast<int (*)[MT * 256]>(smem);
  uint32_t* const words = reinterpret_cast<uint32_t*>(smem + 8 * 2 * STAGE);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int o0 = blockIdx.x * 16;
  const int m0 = blockIdx.y * (MT * 16);
  const int k0 = wave * a.kchunk;
  const int nlines = k0 < a.F ? (min(k0 + a.kchunk, a.F) - k0) >> 7 : 0;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(a.w, 0, a.O * a.F, 0x00020000);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.act), 0, a.M * a.F, 0x00020000);
  // staging: instruction j moves rows 8 j .. 8 j + 7 of the (16 + MT * 16)-row panel
  const int r8 = lane >> 3, piece = (lane & 7) ^ r8;
  int src[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int row = 8 * j + r8;
    const int g = row < 16 ? o0 + row : m0 + row - 16;            // weight row / sample
    const bool in = row < 16 ? g < a.O : g < a.M;
    src[j] = in ? g * a.F + piece * 16 : static_cast<int>(0x80000000u);   // out of range whatever scalar offset is added: zeros
  }
  const unsigned stage0 = lds_addr(smem) + wave * (2 * STAGE);
  auto issue = [&](int line, int buf) {
    const int kb = k0 + line * 128;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const unsigned dst = stage0 + buf * STAGE + j * kFwdInstrBytes;
      const int off = src[j];
      if (j < 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS_AT(dst), 16, off, kb, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, NITI_LDS_AT(dst), 16, off, kb, 0, 0);
    }
  };
  // fragments: lane (row i = lane % 16, 16-byte group kg = lane / 16) of 64-step s reads piece 4 s + kg of row i
  const int fi = lane & 15, kg = lane >> 4;
  const unsigned frow = (fi >> 3) * kFwdInstrBytes + (fi & 7) * 128;
  unsigned fpiece[2];
#pragma unroll
  for (int sstep = 0; sstep < 2; ++sstep) fpiece[sstep] = static_cast<unsigned>(((4 * sstep + kg) ^ (fi & 7)) * 16);
  v4i acc[MT];
  const v4i zero = {0, 0, 0, 0};
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = zero;
  if (nlines > 0) issue(0, 0);
  for (int line = 0; line < nlines; ++line) {
    const int buf = line & 1;
    if (line + 1 < nlines) {
      issue(line + 1, buf ^ 1);
      __builtin_amdgcn_s_waitcnt(0x0F70 | NI);                     // vmcnt(NI): this line has landed, the next one is on its way
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);                          // vmcnt(0)
    }
    const unsigned base = stage0 + buf * STAGE + frow;
    v4i fw[2], fa[MT][2];
#pragma unroll
    for (int sstep = 0; sstep < 2; ++sstep) {
      fw[sstep] = lds_read_b128(base + fpiece[sstep]);
#pragma unroll
      for (int t = 0; t < MT; ++t) fa[t][sstep] = lds_read_b128(base + (2 + 2 * t) * kFwdInstrBytes + fpiece[sstep]);
    }
    lds_settle<0>();
#pragma unroll
    for (int sstep = 0; sstep < 2; ++sstep) {
      asm volatile("" : "+v"(fw[sstep]));
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        asm volatile("" : "+v"(fa[t][sstep]));
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[sstep], fa[t][sstep], acc[t], 0, 0, 0);
      }
    }
  }
  sync_mem();   // every wavefront is done with its stages: the area now takes the partial sums
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][t * 256 + i * 64 + lane] = acc[t][i];
  __syncthreads();
  // wavefront t completes tile t (wavefronts beyond MT only take part in the barriers)
  uint32_t lmax = 0;
  v4i fin = zero;
  if (wave < MT) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < 8; ++w) sum += part[w][wave * 256 + i * 64 + lane];
      fin[i] = sum;
      const uint32_t u = uabs(sum);                        // rows beyond M and columns beyond O are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
  }
  const int shift = grid_shift<8>(a, lmax, words, words + 8);
  if (wave >= MT) return;
  const int m = m0 + wave * 16 + (lane & 15);
  const int ob = o0 + 4 * (lane >> 4);
  if (m >= a.M || ob >= a.O) return;                       // O is a multiple of 4: a dword is inside or outside
  const bool trunc = a.trunc != 0, relu = (a.rq_flags & NITI_RQ_RELU) != 0;
  const long long at = static_cast<long long>(m) * a.O + ob;
  v4i u = zero;
  if (a.method == NITI_ROUND_STOCHASTIC) u = *reinterpret_cast<const v4i*>(a.rand + at);
  int r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[i] = round_any(fin[i], shift, a.method, trunc, u[i]);
    if (relu && r[i] < 0) r[i] = 0;
  }
  *reinterpret_cast<uint32_t*>(a.out8 + at) = pack4_i8(r[0], r[1], r[2], r[3]);
}

// ---- data gradient ------------------------------------------------------------------------------------------
// grid.x = 32-feature tiles of the result, grid.y = groups of 128 samples.  MFMA A = 32 features x 32 reduction steps
// (transposing reads of the staged weight columns), B = 32 samples x 32 steps (error rows): result element 4 g + e of
// a lane is feature 8 g + 4 (lane / 32) + e of sample lane % 32.
__global__ __launch_bounds__(512) void fcw_dgrad_kernel(const FcwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];   // O x 32 bytes, then 4 x 16 x 64 sums; + words
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int f0 = blockIdx.x * 32;
  const int mb = blockIdx.y * 128;
  const int slab = a.O * 32;
  uint32_t* const words = reinterpret_cast<uint32_t*>(smem + (slab > 16384 ? slab : 16384));
  for (int p = tid; p < a.O * 2; p += 512) {
    const int r = p >> 1, half = p & 1;
    *reinterpret_cast<v4i*>(smem + r * 32 + half * 16) = *reinterpret_cast<const v4i*>(a.w + static_cast<long long>(r) * a.F + f0 + half * 16);
  }
  sync_mem();
  const int mt = wave & 3, kh = wave >> 2;
  const int lr = lane & 31, lk = lane >> 5;
  const int j = lane & 15, gg = (lane >> 4) & 1;
  const int m = mb + mt * 32 + lr;
  const bool vm = m < a.M;
  const int8_t* pe = a.err + static_cast<long long>(vm ? m : 0) * a.O + lk * 16;
  const int nsteps = a.O >> 5;                       // O is a multiple of 32
  const int s0 = kh == 0 ? 0 : (nsteps + 1) >> 1;
  const int s1 = kh == 0 ? (nsteps + 1) >> 1 : nsteps;
  const unsigned abase = lds_addr(smem) + (lk * 16 + (j >> 1)) * 32 + gg * 16 + 8 * (j & 1);
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  const v4i zero = {0, 0, 0, 0};
  for (int sb = s0; sb < s1; sb += 4) {               // four steps at a time, their loads in flight together
    v4i fb[4];
    v2i lo[4], hi[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = sb + u;
      fb[u] = (vm && s < s1) ? *reinterpret_cast<const v4i*>(pe + s * 32) : zero;
      const unsigned at = abase + static_cast<unsigned>(min(s, nsteps - 1)) * 1024u;
      lo[u] = lds_read_tr8<0>(at);
      hi[u] = lds_read_tr8<256>(at);
    }
    lds_settle<0>();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const v4i fa = lds_landed(lo[u], hi[u]);
      if (sb + u < s1) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb[u], acc, 0, 0, 0);
    }
  }
  sync_mem();   // every wavefront is done with the weight columns
  int* const park = reinterpret_cast<int*>(smem) + mt * (16 * 64) + lane;
  if (kh == 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) park[e * 64] = acc[e];
  }
  __syncthreads();
  uint32_t lmax = 0;
  if (kh == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      acc[e] += park[e * 64];
      const uint32_t u = uabs(acc[e]);                 // samples beyond M are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
  }
  const int shift = grid_shift<8>(a, lmax, words, words + 8);
  if (kh != 0 || !vm) return;
  const bool trunc = a.trunc != 0;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const long long at = static_cast<long long>(m) * a.F + f0 + 8 * g + 4 * lk;
    v4i u = zero;
    if (a.method == NITI_ROUND_STOCHASTIC) u = *reinterpret_cast<const v4i*>(a.rand + at);
    int r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = round_any(acc[4 * g + e], shift, a.method, trunc, u[e]);
    *reinterpret_cast<uint32_t*>(a.out8 + at) = pack4_i8(r[0], r[1], r[2], r[3]);
  }
}

// ---- data gradient, operands through LDS as whole lines -----------------------------------------------------------
// The kernel above stages 32-byte pieces of the weight rows (a quarter of every line it fetches), takes the error rows
// in 32-byte pieces as well and stores 4-byte pieces.  Here (F and O multiples of 128) a workgroup owns 128 features x
// 32 samples of dx = err w and runs the whole-line product of nn_lines.h over all of O; the sums pass through an LDS
// patch into a row-major arrangement for the rounding.
constexpr int kDgLdsBytes = kLinesLdsBytes + 32 * 4;
__global__ __launch_bounds__(512) void fcw_dgrad_lds_kernel(const FcwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];   // the stages; later 16 KB of parked sums / the 17 KB patch
  uint32_t* const words = reinterpret_cast<uint32_t*>(smem + kLinesLdsBytes);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int f0 = blockIdx.x * 128;
  const int m0 = blockIdx.y * 32;
  const int ft = wave & 3, kh = wave >> 2;
  const int lr = lane & 31, lk = lane >> 5;
  v16i acc = lines_product(a.err, a.w, a.M, a.F, a.O, m0, f0, 0, a.O >> 7, smem);
  lines_add_halves(acc, smem);
  uint32_t lmax = 0;
  if (kh == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint32_t u = uabs(acc[e]);                 // samples beyond M are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
  }
  // The rounding runs in a row-major arrangement - thread (row = tid / 16, piece = tid % 16) takes features
  // 64 q + 4 piece .. + 4 (q = 0, 1) of one sample - so that sixteen lanes read 256 consecutive bytes of random integers;
  // those are requested here, ahead of the range exchange.
  const int row = tid >> 4, p16 = tid & 15;
  const bool rin = m0 + row < a.M;
  const long long at = static_cast<long long>(m0 + row) * a.F + f0 + p16 * 4;
  const v4i zero = {0, 0, 0, 0};
  v4i u[2] = {zero, zero};
  if (a.method == NITI_ROUND_STOCHASTIC && rin) {
#pragma unroll
    for (int q = 0; q < 2; ++q) u[q] = *reinterpret_cast<const v4i*>(a.rand + at + q * 64);
  }
  const int shift = grid_shift<8>(a, lmax, words, words + 8);   // its barriers also retire the parked sums
  const bool trunc = a.trunc != 0;
  constexpr int kPitch = 128 * 4 + 16;
  int8_t* const patch = smem + 16384;                            // [32 samples][128 features] of int32, clear of the parked sums
  if (kh == 0) {
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<v4i*>(patch + lr * kPitch + (ft * 32 + 8 * g + 4 * lk) * 4) = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
  }
  __syncthreads();
  if (!rin) return;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const v4i sum = *reinterpret_cast<const v4i*>(patch + row * kPitch + (q * 64 + p16 * 4) * 4);
    int r[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = round_any(sum[e], shift, a.method, trunc, u[q][e]);
    *reinterpret_cast<uint32_t*>(a.out8 + at + q * 64) = pack4_i8(r[0], r[1], r[2], r[3]);
  }
}

// ---- weight gradient + update -------------------------------------------------------------------------------
// grid.x = 256-feature tiles, grid.y = groups of T 32-row tiles of the weight matrix.  Samples are walked in chunks of
// 128.  MFMA A = 32 features x 32 samples (activation columns), B = 32 output features x 32 samples (error columns):
// result element 4 g + e of a lane is feature 8 g + 4 (lane / 32) + e of output feature lane % 32.
constexpr int kWgActPitch = 256 + 16;   // bytes between samples of the activation tile: eight consecutive samples of
                                        // one 8-byte column fall into eight different bank groups
constexpr int kWgPatchPitch = 32 * 4 + 16;
constexpr int kWgActBytes = 128 * kWgActPitch > 8 * 32 * kWgPatchPitch ? 128 * kWgActPitch : 8 * 32 * kWgPatchPitch;   // tile, then 8 patches

template <int T>
__global__ __launch_bounds__(512) void fcw_wgrad_kernel(const FcwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const act_t = smem;                              // [128 samples][256 features], later 8 patches of 32 x 32 sums
  int8_t* const err_t = smem + kWgActBytes;                // [T][128 samples][32 output features]
  uint32_t* const words = reinterpret_cast<uint32_t*>(err_t + T * 4096);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int f0 = blockIdx.x * 256;
  const int o0 = blockIdx.y * (T * 32);
  const int lk = lane >> 5;
  const int j = lane & 15, gg = (lane >> 4) & 1;
  const v4i zero = {0, 0, 0, 0};
  v16i acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[t][e] = 0;
  const unsigned frag = (lk * 16 + (j >> 1));               // sample inside a 32-step that this lane's address names
  const unsigned abase = lds_addr(act_t) + frag * kWgActPitch + wave * 32 + gg * 16 + 8 * (j & 1);
  const unsigned bbase = lds_addr(err_t) + frag * 32 + gg * 16 + 8 * (j & 1);
  for (int mc = 0; mc < a.M; mc += 128) {
    if (mc > 0) sync_mem();                                 // the previous chunk's tiles have been read
    for (int p = tid; p < 128 * 16; p += 512) {             // activations: 128 samples x 16 pieces of 16 bytes
      const int r = p >> 4, piece = p & 15;
      const int f = f0 + piece * 16;
      v4i v = zero;
      if (mc + r < a.M && f < a.F) v = *reinterpret_cast<const v4i*>(a.act + static_cast<long long>(mc + r) * a.F + f);
      *reinterpret_cast<v4i*>(act_t + r * kWgActPitch + piece * 16) = v;
    }
    for (int p = tid; p < T * 128 * 2; p += 512) {          // errors: T tiles x 128 samples x 2 pieces
      const int t = p / 256, q = p - t * 256;
      const int r = q >> 1, half = q & 1;
      const int o = o0 + t * 32 + half * 16;
      v4i v = zero;
      if (mc + r < a.M && o < a.O) v = *reinterpret_cast<const v4i*>(a.err + static_cast<long long>(mc + r) * a.O + o);
      *reinterpret_cast<v4i*>(err_t + t * 4096 + r * 32 + half * 16) = v;
    }
    sync_mem();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const v2i alo = lds_read_tr8<0>(abase + ks * 32 * kWgActPitch);
      const v2i ahi = lds_read_tr8<8 * kWgActPitch>(abase + ks * 32 * kWgActPitch);
      v2i blo[T], bhi[T];
#pragma unroll
      for (int t = 0; t < T; ++t) {
        blo[t] = lds_read_tr8<0>(bbase + t * 4096 + ks * 1024);
        bhi[t] = lds_read_tr8<256>(bbase + t * 4096 + ks * 1024);
      }
      lds_settle<0>();
      const v4i fa = lds_landed(alo, ahi);
#pragma unroll
      for (int t = 0; t < T; ++t) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, lds_landed(blo[t], bhi[t]), acc[t], 0, 0, 0);
    }
  }
  // ---- out of the MFMA layout: lane (o = tid / 16, piece = tid % 16) takes 16 features of one weight row - with
  // stochastic rounding features 64 q + 4 piece .. + 4 (q = 0 .. 3), so that 16 lanes' random integers are 256
  // consecutive bytes; otherwise 16 piece .. + 16, so that a lane moves 16 bytes of weights at once
  const bool sto = a.method == NITI_ROUND_STOCHASTIC;
  const int lr = lane & 31;
  const int orow = tid >> 4, piece = tid & 15;
  int fin[T][16];
  uint32_t lmax = 0;
  const int src_off = sto ? (piece >> 3) * (32 * kWgPatchPitch) + orow * kWgPatchPitch + (piece & 7) * 16
                          : (piece >> 1) * (32 * kWgPatchPitch) + orow * kWgPatchPitch + (piece & 1) * 64;
  const int src_step = sto ? 2 * 32 * kWgPatchPitch : 16;
#pragma unroll
  for (int t = 0; t < T; ++t) {
    sync_mem();                                              // tiles (or the previous patch) have been read
    int8_t* const patch = act_t + wave * (32 * kWgPatchPitch);
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<v4i*>(patch + lr * kWgPatchPitch + (8 * g + 4 * lk) * 4) =
          v4i{acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
    __syncthreads();
    const int8_t* src = act_t + src_off;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4i v = *reinterpret_cast<const v4i*>(src + q * src_step);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        fin[t][4 * q + e] = v[e];
        const uint32_t u = uabs(v[e]);                       // rows beyond O and columns beyond F are sums of zeros
        lmax = u > lmax ? u : lmax;
      }
    }
  }
  const int shift = grid_shift<8>(a, lmax, words, words + 8);
  const bool trunc = a.trunc != 0;
  if (sto) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int o = o0 + t * 32 + orow;
      if (o >= a.O) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int f = f0 + q * 64 + piece * 4;
        if (f >= a.F) continue;                              // F is a multiple of 16: four features are inside or outside
        const long long at = static_cast<long long>(o) * a.F + f;
        const uint32_t wold = *reinterpret_cast<const uint32_t*>(a.w + at);
        const v4i u = *reinterpret_cast<const v4i*>(a.rand + at);
        int r[4], wn[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          r[e] = round_any(fin[t][4 * q + e], shift, NITI_ROUND_STOCHASTIC, trunc, u[e]);
          const int wo = static_cast<int>(static_cast<int8_t>((wold >> (8 * e)) & 0xFFu));
          wn[e] = clip127(wo - r[e]);
        }
        *reinterpret_cast<uint32_t*>(a.w + at) = pack4_i8(wn[0], wn[1], wn[2], wn[3]);
        if (a.out8 != nullptr) *reinterpret_cast<uint32_t*>(a.out8 + at) = pack4_i8(r[0], r[1], r[2], r[3]);
      }
    }
    return;
  }
  const int f = f0 + piece * 16;
  if (f >= a.F) return;
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int o = o0 + t * 32 + orow;
    if (o >= a.O) continue;
    const long long at = static_cast<long long>(o) * a.F + f;
    const v4i wold = *reinterpret_cast<const v4i*>(a.w + at);
    v4i wnew, g8;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int r[4], wn[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        r[e] = round_any(fin[t][4 * q + e], shift, a.method, trunc, 0);
        const int wo = static_cast<int>(static_cast<int8_t>((static_cast<uint32_t>(wold[q]) >> (8 * e)) & 0xFFu));
        wn[e] = clip127(wo - r[e]);
      }
      wnew[q] = static_cast<int>(pack4_i8(wn[0], wn[1], wn[2], wn[3]));
      g8[q] = static_cast<int>(pack4_i8(r[0], r[1], r[2], r[3]));
    }
    *reinterpret_cast<v4i*>(a.w + at) = wnew;
    if (a.out8 != nullptr) *reinterpret_cast<v4i*>(a.out8 + at) = g8;
  }
}

int resident_blocks(const void* kernel, int threads, size_t lds) {
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds) != hipSuccess)
    return 0;
  return cus * per_cu;
}

constexpr int kMaxSlots = 4096;

// forward: reduction elements per wavefront (a multiple of 256), sixteen wavefronts per tile
int fwd_chunk(int F) { return ((F + 15) / 16 + 255) / 256 * 256; }
size_t fwd_lds(int mt) { return static_cast<size_t>(16) * mt * 256 * 4 + 32 * 4; }
size_t dgrad_lds(int O) { return static_cast<size_t>(O * 32 > 16384 ? O * 32 : 16384) + 32 * 4; }
size_t wgrad_lds(int t) { return static_cast<size_t>(kWgActBytes) + static_cast<size_t>(t) * 4096 + 32 * 4; }

bool shape_ok(int which, int M, int O, int F) {
  if (M <= 0 || O <= 0 || F <= 0) return false;
  if (static_cast<long long>(M) * F >= 0x7fffffffLL || static_cast<long long>(O) * F >= 0x7fffffffLL) return false;
  if (which == NITI_FC_FORWARD) return F % 16 == 0 && O % 4 == 0;
  if (which == NITI_FC_DGRAD) return O % 32 == 0 && F % 32 == 0 && O <= 4096;
  if (which == NITI_FC_WGRAD) return O % 16 == 0 && F % 16 == 0;
  return false;
}

template <class K>
int resident_cached(int (&cache)[kDeviceSlots], K kernel, int threads, size_t lds) {
  int& r = cache[device_slot()];
  if (r == 0) {
    if (lds > 48 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return 0;
    r = resident_blocks(reinterpret_cast<const void*>(kernel), threads, lds);
  }
  return r;
}

size_t fwd_lds_bytes(int mt) { return static_cast<size_t>(16) * (2 + 2 * mt) * kFwdInstrBytes + 32 * 4; }
// workgroups of the LDS-staged forward kernel the device holds at once (MT = 1, 2)
int fwd_lds_resident(int mt) {
  static int c1[kDeviceSlots] = {}, c2[kDeviceSlots] = {};
  if (mt == 1) return resident_cached(c1, fcw_fwd_lds_kernel<1>, 512, fwd_lds_bytes(1));
  return resident_cached(c2, fcw_fwd_lds_kernel<2>, 512, fwd_lds_bytes(2));
}
int fwd_resident(int mt) {
  static int c1[kDeviceSlots] = {}, c2[kDeviceSlots] = {}, c4[kDeviceSlots] = {};
  if (mt == 1) return resident_cached(c1, fcw_fwd_kernel<1>, 1024, fwd_lds(1));
  if (mt == 2) return resident_cached(c2, fcw_fwd_kernel<2>, 1024, fwd_lds(2));
  return resident_cached(c4, fcw_fwd_kernel<4>, 1024, fwd_lds(4));
}
int wgrad_resident(int t) {
  static int c1[kDeviceSlots] = {}, c2[kDeviceSlots] = {}, c4[kDeviceSlots] = {};
  if (t == 1) return resident_cached(c1, fcw_wgrad_kernel<1>, 512, wgrad_lds(1));
  if (t == 2) return resident_cached(c2, fcw_wgrad_kernel<2>, 512, wgrad_lds(2));
  return resident_cached(c4, fcw_wgrad_kernel<4>, 512, wgrad_lds(4));
}

int dgrad_lds_resident() {
  static int c[kDeviceSlots] = {};
  return resident_cached(c, fcw_dgrad_lds_kernel, 512, static_cast<size_t>(kDgLdsBytes));
}
// workgroups of the whole-line data-gradient kernel for this shape, or 0 when the other kernel runs it
long long dgrad_lds_blocks(int M, int O, int F) {
  if (F % 128 != 0 || O % 128 != 0) return 0;
  const char* e = getenv("NITI_FC_LDS");
  if (e != nullptr && e[0] == '0') return 0;
  const long long nb = static_cast<long long>(F / 128) * ((M + 31) / 32);
  return (nb <= kMaxSlots && nb <= dgrad_lds_resident()) ? nb : 0;
}
int dgrad_resident(int O) {
  static int attr_of[kDeviceSlots] = {};
  int& attr = attr_of[device_slot()];
  const size_t lds = dgrad_lds(O);
  if (attr < static_cast<int>(lds)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(fcw_dgrad_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)) != hipSuccess)
      return 0;
    attr = static_cast<int>(lds);
  }
  return resident_blocks(reinterpret_cast<const void*>(fcw_dgrad_kernel), 512, lds);
}

// Workgroups of the launch on the current device and the per-workgroup tile count (MT / T); 0 when the shape is outside
// the kernels or no variant's grid fits on the device at once.
long long plan(int which, int M, int O, int F, int* tiles) {
  *tiles = 0;
  if (!shape_ok(which, M, O, F)) return 0;
  if (which == NITI_FC_DGRAD) {
    if (const long long nl = dgrad_lds_blocks(M, O, F)) {
      *tiles = 1;
      return nl;
    }
    const long long nb = static_cast<long long>(F / 32) * ((M + 127) / 128);
    *tiles = 1;
    return (nb <= kMaxSlots && nb <= dgrad_resident(O)) ? nb : 0;
  }
  // NITI_FC_TILES pins the tiles per workgroup (measurements); otherwise the smallest count whose grid fits
  const char* e = getenv("NITI_FC_TILES");
  const int pin = e != nullptr ? atoi(e) : 0;
  const bool fwd = which == NITI_FC_FORWARD;
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 256;
  long long best = 0;
  for (int t = 1; t <= 4; t *= 2) {
    if (pin != 0 && t != pin) continue;
    const long long nb = fwd ? static_cast<long long>((O + 15) / 16) * ((M + 16 * t - 1) / (16 * t))
                             : static_cast<long long>((F + 255) / 256) * ((O + 32 * t - 1) / (32 * t));
    if (nb > kMaxSlots || nb > (fwd ? fwd_resident(t) : wgrad_resident(t))) continue;
    // forward: more sample tiles per workgroup re-read the weights less often, as long as every compute unit still
    // gets a workgroup (measured on 128 x 8192 x 1024: 21.7 / 15.9 / 23.3 us for 1 / 2 / 4 tiles)
    if (best == 0 || (fwd && nb >= cus)) {
      best = nb;
      *tiles = t;
    }
  }
  return best;
}

}  // namespace
}  // namespace niti

using namespace niti;

extern "C" size_t niti_linear_i8_sync_words(int which, int M, int O, int F) {
  int tiles = 0;
  const long long nb = plan(which, M, O, F, &tiles);
  return nb == 0 ? 0 : static_cast<size_t>(kSlot0) + slot_words(static_cast<int>(nb));
}

static int fcw_common(const char* who, int which, FcwArgs& a, int M, int O, int F, int target_bits, int method, int div_mode,
                      int bw_mode, const int32_t* rand, uint32_t* sync, size_t sync_words, int32_t* shift_out,
                      const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out) {
  clear_error();
  if (M <= 0 || O <= 0 || F <= 0) return fail(NITI_ERR_INVALID_ARG, "%s: non-positive extent", who);
  if (sync == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (target_bits < 1 || target_bits > 7) return fail(NITI_ERR_INVALID_ARG, "%s: target_bits=%d outside 1..7", who, target_bits);
  if (method != NITI_ROUND_NEAREST && method != NITI_ROUND_PSEUDO_STOCHASTIC && method != NITI_ROUND_STOCHASTIC)
    return fail(NITI_ERR_INVALID_ARG, "%s: rounding method %d", who, method);
  if (method == NITI_ROUND_STOCHASTIC && (rand == nullptr || !aligned16(rand)))
    return fail(NITI_ERR_INVALID_ARG, "%s: stochastic rounding needs `rand` (16-byte aligned, one int32 per output element)", who);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "%s: div_mode=%d", who, div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "%s: bw_mode=%d", who, bw_mode);
  if (!shape_ok(which, M, O, F)) return fail(NITI_ERR_UNSUPPORTED, "%s: M=%d O=%d F=%d outside these kernels; use the GEMM entry point", who, M, O, F);
  const size_t need = niti_linear_i8_sync_words(which, M, O, F);
  if (need == 0) return fail(NITI_ERR_UNSUPPORTED, "%s: the workgroups of M=%d O=%d F=%d do not fit on the device at once", who, M, O, F);
  if (sync_words < need) return fail(NITI_ERR_WORKSPACE, "%s: needs %zu zeroed sync words, got %zu", who, need, sync_words);
  a.sync = sync;
  a.rand = rand;
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

extern "C" int niti_linear_i8_fwd_requant(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int target_bits,
                                          int method, int div_mode, int bw_mode, unsigned rq_flags, const int32_t* rand,
                                          uint32_t* sync, size_t sync_words, int32_t* shift_out, const int32_t* exp_a,
                                          const int32_t* exp_b, int32_t* exp_out, void* stream) {
  FcwArgs a{};
  const char* who = "linear_fwd_requant";
  int st = fcw_common(who, NITI_FC_FORWARD, a, M, O, F, target_bits, method, div_mode, bw_mode, rand, sync, sync_words, shift_out,
                      exp_a, exp_b, exp_out);
  if (st != NITI_OK) return st;
  if (act == nullptr || w == nullptr || out8 == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (!aligned16(act) || !aligned16(w) || reinterpret_cast<uintptr_t>(out8) % 4 != 0) return fail(NITI_ERR_INVALID_ARG, "%s: misaligned pointer", who);
  if ((rq_flags & ~NITI_RQ_RELU) != 0u) return fail(NITI_ERR_INVALID_ARG, "%s: rq_flags=%#x", who, rq_flags);
  a.act = act;
  a.w = const_cast<int8_t*>(w);
  a.out8 = out8;
  a.rq_flags = rq_flags;
  a.kchunk = fwd_chunk(F);
  int mt = 0;
  plan(NITI_FC_FORWARD, M, O, F, &mt);
  const dim3 grid((O + 15) / 16, (M + 16 * mt - 1) / (16 * mt));
  hipStream_t s = static_cast<hipStream_t>(stream);
  // whole lines through LDS where the rows are whole lines (NITI_FC_LDS=0 pins the direct-fragment kernel)
  const char* e = getenv("NITI_FC_LDS");
  if (F % 128 == 0 && mt <= 2 && (e == nullptr || e[0] != '0') && static_cast<long long>(grid.x) * grid.y <= fwd_lds_resident(mt)) {
    a.kchunk = ((F + 7) / 8 + 127) / 128 * 128;
    if (mt == 1) hipLaunchKernelGGL(fcw_fwd_lds_kernel<1>, grid, dim3(512), fwd_lds_bytes(1), s, a);
    else hipLaunchKernelGGL(fcw_fwd_lds_kernel<2>, grid, dim3(512), fwd_lds_bytes(2), s, a);
    return check_launch(who);
  }
  if (mt == 1) hipLaunchKernelGGL(fcw_fwd_kernel<1>, grid, dim3(1024), fwd_lds(1), s, a);
  else if (mt == 2) hipLaunchKernelGGL(fcw_fwd_kernel<2>, grid, dim3(1024), fwd_lds(2), s, a);
  else hipLaunchKernelGGL(fcw_fwd_kernel<4>, grid, dim3(1024), fwd_lds(4), s, a);
  return check_launch(who);
}

extern "C" int niti_linear_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int M, int O, int F, int target_bits,
                                            int method, int div_mode, int bw_mode, const int32_t* rand, uint32_t* sync,
                                            size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                            int32_t* exp_out, void* stream) {
  FcwArgs a{};
  const char* who = "linear_dgrad_requant";
  int st = fcw_common(who, NITI_FC_DGRAD, a, M, O, F, target_bits, method, div_mode, bw_mode, rand, sync, sync_words, shift_out,
                      exp_a, exp_b, exp_out);
  if (st != NITI_OK) return st;
  if (err == nullptr || w == nullptr || dx8 == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (!aligned16(err) || !aligned16(w) || reinterpret_cast<uintptr_t>(dx8) % 4 != 0) return fail(NITI_ERR_INVALID_ARG, "%s: misaligned pointer", who);
  a.err = err;
  a.w = const_cast<int8_t*>(w);
  a.out8 = dx8;
  if (dgrad_lds_blocks(M, O, F) != 0) {
    if (!aligned16(dx8)) return fail(NITI_ERR_INVALID_ARG, "%s: misaligned pointer", who);
    hipLaunchKernelGGL(fcw_dgrad_lds_kernel, dim3(F / 128, (M + 31) / 32), dim3(512), static_cast<size_t>(kDgLdsBytes),
                       static_cast<hipStream_t>(stream), a);
    return check_launch(who);
  }
  const size_t lds = dgrad_lds(O);
  hipLaunchKernelGGL(fcw_dgrad_kernel, dim3(F / 32, (M + 127) / 128), dim3(512), lds, static_cast<hipStream_t>(stream), a);
  return check_launch(who);
}

extern "C" int niti_linear_i8_wgrad_update(const int8_t* err, const int8_t* act, int8_t* w, int M, int O, int F, int mu, int method,
                                           int div_mode, int bw_mode, const int32_t* rand, uint32_t* sync, size_t sync_words,
                                           int8_t* g8_out, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                           int32_t* exp_out, void* stream) {
  FcwArgs a{};
  const char* who = "linear_wgrad_update";
  int st = fcw_common(who, NITI_FC_WGRAD, a, M, O, F, mu, method, div_mode, bw_mode, rand, sync, sync_words, shift_out, exp_a, exp_b,
                      exp_out);
  if (st != NITI_OK) return st;
  if (err == nullptr || act == nullptr || w == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (!aligned16(err) || !aligned16(act) || !aligned16(w) || !aligned16(g8_out)) return fail(NITI_ERR_INVALID_ARG, "%s: misaligned pointer", who);
  a.err = err;
  a.act = act;
  a.w = w;
  a.out8 = g8_out;
  int t_use = 0;
  plan(NITI_FC_WGRAD, M, O, F, &t_use);
  const dim3 grid((F + 255) / 256, (O + 32 * t_use - 1) / (32 * t_use));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (t_use == 1) hipLaunchKernelGGL(fcw_wgrad_kernel<1>, grid, dim3(512), wgrad_lds(1), s, a);
  else if (t_use == 2) hipLaunchKernelGGL(fcw_wgrad_kernel<2>, grid, dim3(512), wgrad_lds(2), s, a);
  else hipLaunchKernelGGL(fcw_wgrad_kernel<4>, grid, dim3(512), wgrad_lds(4), s, a);
  return check_launch(who);
}
