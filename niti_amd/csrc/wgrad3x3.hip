// Native int8 weight gradient of a 3x3, stride-1, pad-1 convolution on the gfx950 matrix cores:
//   dw[k,r,s,c] = sum_{n,p,q} err[n,p,q,k] * act[n,p+r-1,q+s-1,c]
//
// GEMM view: rows = output channels k, columns = (tap, input channel c), reduction over the
// output pixels.  Both operands are stored with channels contiguous and the reduction index
// (pixels) strided, the opposite of what an MFMA operand needs (16 reduction bytes per lane).
// The kernel therefore stages tiles in their natural [pixel][channel] layout with
// buffer_load ... lds and builds the fragments with ds_read_b64_tr_b8, the gfx950 transposing
// LDS read: within 16 lanes, lane j supplies the address of an 8-byte row and lane i receives
// byte (i % 8) of the rows supplied by lanes 2m + i/8 (m = 0..7).  Pointing lanes 2m and 2m+1 at
// the two 8-channel halves of pixel m gives every lane 8 consecutive pixels of channel i.
//
// Work split: a workgroup (8 wavefronts, 4 x 2) owns 128 output channels x 64 input channels x 9
// taps of accumulators (one 32 x 32 tile per tap and wavefront: 144 registers per lane, two
// wavefronts per SIMD) and walks over "bands" of 128 consecutive output pixels
// (whole rows of an image, or whole small images).  Per band it stages the 128 x 128 error tile
// and the activation rows with their halo once, and serves all nine taps from that one halo
// tile, so activations are read from L2 once instead of nine times.  The pixel range is split
// over gridDim.z workgroups; each writes its partial sums to a workspace slice and a second
// kernel adds the slices (integer addition: any split gives the same result).  The arrangement with
// 128 x 32 tiles (wgrad3x3_narrow_kernel) can also add the slices itself, at the end of the same
// launch, once all of its workgroups - resident together - have written theirs.
#include <stdlib.h>

#include <type_traits>

#include "common.h"
#include "lds_asm.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kOob = -1;

template <int N>
__device__ inline void wg_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (((N >> 4) & 3) << 14) | 0x0F70);
}
__device__ inline void wg_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

struct WgradArgs {
  const int8_t* act;  // [N,H,W,C], H == W == Q
  const int8_t* err;  // [N,Q,Q,K]
  int32_t* partial;   // [splits][slice_stride], slice z holds K*9*C partial sums
  long long slice_stride;
  int N, C, K;
  int Cp;             // gradient columns (input channels) kept per tap in the partial sums: C, or fewer when the rest is padding
  int bands, bands_per_split;
  long long act_bytes, err_bytes;
};

// Workgroups are handed to the eight accelerator dies (each with its own L2) round robin in launch order.  The
// workgroups that read the same pixels - all tiles of one pixel range - should share a die: workgroup p of the
// launch therefore takes the work item (p % 8) * (total / 8) + p / 8 of the order "tiles fastest, pixel ranges
// slowest", which gives every die a contiguous run of that order.  (A mapping for locality only: any assignment
// of work items to workgroups computes the same sums.)
struct WorkItem { int x, y, z; };
__device__ inline WorkItem die_local_work_item() {
  const int gx = gridDim.x, gy = gridDim.y, gz = gridDim.z;
  const int total = gx * gy * gz;
  int p = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
  if (total % 8 == 0) p = (p % 8) * (total / 8) + p / 8;
  WorkItem w;
  w.x = p % gx;
  p /= gx;
  w.y = p % gy;
  w.z = p / gy;
  return w;
}

// One stage of the main loop: KS reduction steps of 32 pixels x three filter rows x three taps, all fragments by
// transposing LDS reads.  The reads are inline assembly (see lds_asm.h: the builtin form would wait for the loads
// of the following stages, just issued, before every read) and run one filter row ahead of the MFMAs: row i + 1 is
// requested, then the wait leaves exactly those requests in flight, then row i multiplies.
// a_base: error-tile offsets of the lane's two 8-byte rows (reduction step 0); b_base: halo-tile offsets of its rows
// (reduction step 0, filter row 0); ROWB: bytes of a halo row.  kShiftTaps: the second and third tap of a filter row
// are byte shifts of the first one's pixel sequence (rows of at least 8 pixels), otherwise every tap is read.
// kShiftErr (rows of 8 or 16 pixels, which lie whole inside a lane's 16 pixels): the ERROR fragment is shifted instead -
// sum_q err[q] act[q+s-1] = sum_q' err[q'-s+1] act[q'] -, once per reduction step for all three filter rows (8 byte
// shifts instead of 24 per nine MFMAs), and every filter row reads one aligned activation fragment (b_base then names
// the pixels themselves, halo column + 1): 8 instead of 11 LDS reads.
// behind_first: run once behind the first step's products - the caller's load instructions for a later stage.  A
// wavefront issues in order and the memory pipeline takes a few hundred clocks to accept a stage's loads; right behind
// the stage barrier all eight wavefronts would spend them at the same time with nothing queued on the matrix units.
template <int Q, int BR, int HR, int ROWB, bool kShiftTaps, int NB, bool kShiftErr = false, int KS = 4, class F>
__device__ inline void wgrad_stage(unsigned sbase, const int (&a_base)[2], const int (&b_base)[NB], v16i (&acc)[9], F&& behind_first) {
  v2i alo[2], ahi[2];   // [reduction step & 1]
  v2i rd[2][NB];        // [row step & 1]
  v4i af[2];
  auto request = [&](auto stepc) {
    constexpr int step = decltype(stepc)::value;
    constexpr int ks = step / 3, r = step % 3;
    constexpr int prow = ks * 32 / Q;                         // first output row of this reduction step inside the tile
    constexpr int hrow0 = (prow / BR) * HR + (prow % BR);     // its halo row for filter row 0
    if constexpr (r == 0) {
      alo[ks & 1] = lds_read_tr8<ks * 4096>(sbase + a_base[0]);
      ahi[ks & 1] = lds_read_tr8<ks * 4096>(sbase + a_base[1]);
    }
#pragma unroll
    for (int q = 0; q < NB; ++q) rd[step & 1][q] = lds_read_tr8<(hrow0 + r) * ROWB>(sbase + b_base[q]);
  };
  request(std::integral_constant<int, 0>{});
  static_for<3 * KS>([&](auto stepc) {
    constexpr int step = decltype(stepc)::value;
    constexpr int ks = step / 3, r = step % 3;
    if constexpr (step + 1 < 3 * KS) request(std::integral_constant<int, step + 1>{});
    lds_settle<(step + 1 < 3 * KS) ? NB + ((step + 1) % 3 == 0 ? 2 : 0) : 0>();
    if constexpr (r == 0) af[ks & 1] = lds_landed(alo[ks & 1], ahi[ks & 1]);
    v2i (&d)[NB] = rd[step & 1];
#pragma unroll
    for (int q = 0; q < NB; ++q) asm volatile("" : "+v"(d[q]));
    const v4i a4 = af[ks & 1];
    if constexpr (kShiftErr) {
      static_assert(NB == 2 && (Q == 8 || Q == 16));
      const v4i bf = {d[0][0], d[0][1], d[1][0], d[1][1]};
      // err[q'+1] (tap 0) and err[q'-1] (tap 2) of the lane's 16 pixels, zero where the row ends
      const uint32_t l0 = static_cast<uint32_t>(a4[0]), l1 = static_cast<uint32_t>(a4[1]), h0 = static_cast<uint32_t>(a4[2]),
                     h1 = static_cast<uint32_t>(a4[3]);
      v4i aL, aR;
      aL[0] = static_cast<int>(__builtin_amdgcn_alignbyte(l1, l0, 1));
      aL[1] = static_cast<int>(Q == 16 ? __builtin_amdgcn_alignbyte(h0, l1, 1) : l1 >> 8);
      aL[2] = static_cast<int>(__builtin_amdgcn_alignbyte(h1, h0, 1));
      aL[3] = static_cast<int>(h1 >> 8);
      aR[0] = static_cast<int>(l0 << 8);
      aR[1] = static_cast<int>(__builtin_amdgcn_alignbyte(l1, l0, 3));
      aR[2] = static_cast<int>(Q == 16 ? __builtin_amdgcn_alignbyte(h0, l1, 3) : h0 << 8);
      aR[3] = static_cast<int>(__builtin_amdgcn_alignbyte(h1, h0, 3));
      acc[r * 3 + 0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aL, bf, acc[r * 3 + 0], 0, 0, 0);
      acc[r * 3 + 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, bf, acc[r * 3 + 1], 0, 0, 0);
      acc[r * 3 + 2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aR, bf, acc[r * 3 + 2], 0, 0, 0);
    } else if constexpr (!kShiftTaps) {
#pragma unroll
      for (int s = 0; s < 3; ++s)
        acc[r * 3 + s] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, v4i{d[2 * s][0], d[2 * s][1], d[2 * s + 1][0], d[2 * s + 1][1]},
                                                               acc[r * 3 + s], 0, 0, 0);
    } else {
      // the byte sequences the two 8-pixel halves are cut from: [d0 d1 d2] and [e0 e1 e2] (dwords)
      const int d0 = d[0][0], d1 = d[0][1], d2 = d[1][0];
      const int e0 = Q >= 16 ? d[1][0] : d[2][0], e1 = Q >= 16 ? d[1][1] : d[2][1];
      const int e2 = d[NB - 1][0];
      acc[r * 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, v4i{d0, d1, e0, e1}, acc[r * 3], 0, 0, 0);
#pragma unroll
      for (int s = 1; s < 3; ++s) {
        const v4i bf = {static_cast<int>(__builtin_amdgcn_alignbyte(d1, d0, s)), static_cast<int>(__builtin_amdgcn_alignbyte(d2, d1, s)),
                        static_cast<int>(__builtin_amdgcn_alignbyte(e1, e0, s)), static_cast<int>(__builtin_amdgcn_alignbyte(e2, e1, s))};
        acc[r * 3 + s] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, bf, acc[r * 3 + s], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);   // the next row's requests and wait stay behind these products
    if constexpr (step == 0) {
      behind_first();
      __builtin_amdgcn_sched_barrier(0);
    }
  });
}

// Q: image width = height; BR: output rows of one image per band; NI: images per band; BR*NI*Q == 128
template <int Q, int BR, int NI>
struct Geom {
  static constexpr int RP = (Q + 2 + 15) / 16 * 16;  // halo row pitch in pixel slots (multiple of 16)
  static constexpr int HR = BR + 2;                   // halo rows per image
  static constexpr int ACT_INSTR = NI * HR * (RP / 16);
  static constexpr int ACT_BYTES = NI * HR * RP * 64;
  static constexpr int ERR_BYTES = 128 * 128;
  static constexpr int STAGE_BYTES = ERR_BYTES + ACT_BYTES;
  static constexpr int ACT_LOADS = (ACT_INSTR + 7) / 8;  // per wavefront
  static constexpr int NL = 2 + ACT_LOADS;               // loads per wavefront per stage
  static constexpr int BANDS_PER_IMAGE = Q / BR;         // valid when NI == 1
  static_assert(BR * NI * Q == 128, "a band is 128 output pixels");
};

template <int Q, int BR, int NI, int STAGES>
__global__ __launch_bounds__(512, 1) void wgrad3x3_kernel(const WgradArgs a) {
  using G = Geom<Q, BR, NI>;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];  // STAGES stages + 1 KB dump slot
  int8_t* const dump = smem + STAGES * G::STAGE_BYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const WorkItem item = die_local_work_item();
  const int k0 = item.x * 128;
  const int c0 = item.y * 64;
  const int band_begin = item.z * a.bands_per_split;
  const int band_end = min(band_begin + a.bands_per_split, a.bands);
  const int nb = band_end - band_begin;

  const __amdgpu_buffer_rsrc_t ract = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.act), 0, a.act_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rerr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.err), 0, a.err_bytes, 0x00020000);

  // ---- staging.  Error tile: 16 instructions of 8 pixels x 128 bytes; lane -> (pixel lane/8, piece lane%8)
  int err_off[2];  // byte offset of this lane's 16 bytes relative to the band's first pixel, or kOob
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int pix = (wave + 8 * i) * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((pix >> 1) & 7);
    const int ch = k0 + piece * 16;
    err_off[i] = ch < a.K ? pix * a.K + ch : kOob;
  }
  // Activation halo tile: NI images x HR rows x RP pixel slots x 64 bytes; an instruction fills 16 slots
  int act_off[G::ACT_LOADS];   // byte offset relative to the band's first image row p0 = 0, or kOob
  int act_hrow[G::ACT_LOADS];  // halo row (to test against the image border per band)
  int act_dst[G::ACT_LOADS];   // LDS byte offset of the instruction's 1 KB inside the stage, or -1 -> dump
#pragma unroll
  for (int i = 0; i < G::ACT_LOADS; ++i) {
    const int idx = wave + 8 * i;
    int off = kOob, hrow = 0, dst = -1;
    if (idx < G::ACT_INSTR) {
      const int ni = idx / (G::HR * (G::RP / 16));
      const int rem = idx - ni * (G::HR * (G::RP / 16));
      const int h = rem / (G::RP / 16);
      const int wg = rem - h * (G::RP / 16);
      const int w = wg * 16 + (lane >> 2);
      const int piece = (lane & 3) ^ ((w >> 2) & 3);
      const int ch = c0 + piece * 16;
      const int iw = w - 1;
      hrow = h;
      dst = G::ERR_BYTES + ((ni * G::HR + h) * G::RP + wg * 16) * 64;
      if (iw >= 0 && iw < Q && ch < a.C) off = ((ni * Q + (h - 1)) * Q + iw) * a.C + ch;  // relative to image n0, row p0
      else off = kOob;
      if (w >= Q + 2) off = kOob;
    }
    act_off[i] = off;
    act_hrow[i] = hrow;
    act_dst[i] = dst;
  }

  auto issue = [&](int band, int st) {
    int8_t* base = smem + st * G::STAGE_BYTES;
    const int pixbase = band * 128;  // first output pixel of the band in [N*Q*Q]
    // image / first row of the band
    const int n0 = pixbase / (Q * Q);
    const int p0 = (pixbase - n0 * (Q * Q)) / Q;
    const int eb = pixbase * a.K;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int off = err_off[i] == kOob ? kOob : eb + err_off[i];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rerr, NITI_LDS(base + (wave + 8 * i) * 1024), 16, off, 0, 0, 0);
    }
    const int ab = (n0 * Q + p0) * Q * a.C;
#pragma unroll
    for (int i = 0; i < G::ACT_LOADS; ++i) {
      const int ih = p0 + act_hrow[i] - 1;
      const bool ok = act_off[i] != kOob && ih >= 0 && ih < Q;
      const int off = ok ? ab + act_off[i] : kOob;
      int8_t* dst = act_dst[i] >= 0 ? base + act_dst[i] : dump;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ract, NITI_LDS(dst), 16, off, 0, 0, 0);
    }
  };

  // ---- fragment addressing (transposing LDS reads)
  const int j = lane & 15;         // lane inside its group of 16
  const int gg = (lane >> 4) & 1;  // which 16 channels of the 32-row MFMA operand
  const int lk = lane >> 5;        // which 16 of the 32 pixels of a reduction step
  const int wk = wave & 3;         // 32-output-channel quarter of the tile
  const int wc = wave >> 2;        // 32-input-channel half of the tile
  int a_base[2];     // [o]: error tile byte offset of this lane's 8-byte row, reduction step 0
  // Activation fragments: a lane holds 16 consecutive pixels (bytes) of one channel.  The three taps of a filter
  // row read windows that start 0, 1 and 2 slots into the halo row, so only the window of the first tap is read
  // from LDS, together with the 8 slots that follow it, and the other two are byte shifts of that sequence
  // (v_alignbyte).  With 8-pixel image rows the two halves of a fragment lie in different rows and each half
  // gets its own following slots.
  constexpr int NB = Q >= 16 ? 3 : 4;
  int b_base[NB];    // halo tile byte offsets of this lane's 8-byte rows, reduction step 0, filter row 0
#pragma unroll
  for (int o = 0; o < 2; ++o) {
    const int lpix = 16 * lk + 8 * o + (j >> 1);  // pixel inside the 32-pixel step
    const int cb = wk * 32 + gg * 16 + 8 * (j & 1);
    a_base[o] = lpix * 128 + ((((cb >> 4) ^ ((lpix >> 1) & 7)) << 4) | (cb & 15));
  }
  {
    const int cb = wc * 32 + gg * 16 + 8 * (j & 1);
    auto slot_addr = [&](int lrow, int w) {
      return G::ERR_BYTES + (lrow * G::RP + w) * 64 + ((((cb >> 4) ^ ((w >> 2) & 3)) << 4) | (cb & 15));
    };
    const int p0 = 16 * lk + (j >> 1), p1 = p0 + 8;   // pixels of the two halves inside the 32-pixel step
    if (Q >= 16) {
      b_base[0] = slot_addr(p0 / Q, p0 % Q);
      b_base[1] = slot_addr(p1 / Q, p1 % Q);
      b_base[2] = slot_addr(p0 / Q, p0 % Q + 16);
    } else {
      b_base[0] = slot_addr(p0 / Q, p0 % Q);
      b_base[1] = slot_addr(p0 / Q, p0 % Q + 8);
      b_base[2] = slot_addr(p1 / Q, p1 % Q);
      b_base[NB - 1] = slot_addr(p1 / Q, p1 % Q + 8);
    }
  }

  v16i acc[9];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[t][e] = 0;

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < nb) issue(band_begin + s, s);

  for (int it = 0; it < nb; ++it) {
    if (it + STAGES - 2 < nb) wg_wait_vmcnt<(STAGES - 2) * G::NL>();
    else wg_wait_vmcnt<0>();
    wg_sync();
    wgrad_stage<Q, BR, G::HR, G::RP * 64, true, NB>(lds_addr(smem + (it % STAGES) * G::STAGE_BYTES), a_base, b_base, acc, [&] {
      if (it + STAGES - 1 < nb) issue(band_begin + it + STAGES - 1, (it + STAGES - 1) % STAGES);
    });
  }

  // ---- partial sums: acc[t][4g+e] = dw[k0+wk*32+8g+4*lk+e][tap t][c0+wc*32+(lane&31)]
  int32_t* out = a.partial + static_cast<long long>(item.z) * a.slice_stride;
  const int c = c0 + wc * 32 + (lane & 31);
  if (c < a.Cp) {
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = k0 + wk * 32 + g * 8 + lk * 4 + e;
        if (k >= a.K) continue;
#pragma unroll
        for (int t = 0; t < 9; ++t) out[(static_cast<long long>(k) * 9 + t) * a.Cp + c] = acc[t][4 * g + e];
      }
  }
}

// Partial sums -> rounded gradient -> updated weights in one launch (the int32 gradient is not stored unless
// asked for).  A workgroup owns kFinishV x 64 int4 columns at a grid-wide stride; its NW wavefronts each add every
// NW-th slice of every column (no barrier in between, so all those loads are in flight together), column v is
// then completed through LDS by wavefront v % NW, which keeps the sums in registers.  The workgroup publishes its
// largest magnitude in its slot and waits for the slots of all workgroups (all resident: the host sizes the grid
// for that; the wait is bounded by a wall-clock limit), derives the shift from the maximum over the slots, and
// every wavefront applies w = clip(w - round(sum >> shift)) to its columns.  NW = 16 serves the launches with
// many slices and few columns, NW = 4 the others.
constexpr int kFinishV = 16;
constexpr int kFusedV = 48;         // columns per lane in the one-launch form (8 wavefronts: six each)
constexpr int kArriveSlots = 256;   // workgroups of the one-launch form at most
constexpr uint32_t kPartialBias = 1u << 23;   // added to the partial sums of the one-launch form before they are cut to 24 bits
constexpr int kFinishSlot0 = 16;
struct FinishArgs {
  const int32_t* partial;
  long long slice_stride;
  int splits;
  long long nv;        // int4 columns of the gradient: K*9*C / 4
  int C, Cw;           // channels per gradient row / per weight row (Cw <= C; the rest is channel padding)
  int8_t* w;           // [K][9][Cw], updated in place
  int8_t* g8;          // optional rounded gradient, laid out like w
  int32_t* dw;         // optional int32 gradient [K][9][C]
  int8_t* wprep;       // optional: the halo convolution kernel's forward copy of the [K][9][C] filter, kept in step with w
  uint32_t* sync;      // word 0: max |sum| (output); word 1: wait gave up; words kFinishSlot0..: slots, zero on entry
  int roundtrip, target_bits, method, trunc, bw_mode;
  int predict;         // *shift_out holds a predicted shift on entry
  long long spin_limit;
  uint32_t* sticky;    // device-wide word set when the wait gives up, may be null
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
  uint32_t* arrive;    // one-launch form only: a slot per workgroup, zero on entry, filled when its partial sums are in memory
  // one-launch form only.  A slice then holds, per group of four consecutive output channels kg, tap t and input channel
  // c (unit u = (kg * 9 + t) * C + c), three planes: bits 0..15 of the four sums (8 bytes at 8u), bits 16..23 (4 bytes at
  // units * 8 + 4u) and bits 24..31 (4 bytes at units * 12 + 4u).  The third plane is written only by a workgroup whose
  // sums do not fit 24 bits; it says so in wide[tile + tiles * slice] (zero on entry) and in the value of its arrival slot.
  uint32_t* wide;
  int tiles_k, tiles_c;
};

typedef unsigned int v2u __attribute__((ext_vector_type(2)));

template <int NW>
struct FinishShared {
  v4i part[2][NW][64];
  uint32_t wmax[NW];
  uint32_t gshare;
};

// The finishing pass of workgroup `block` out of `nblocks` (V = int4 columns per lane it may own, NW its wavefronts).
// predicted_raw: the word read from a.shift_out (or anything when there is no prediction) at kernel start.
// any_wide (uniform): some workgroup wrote the third plane (top bytes) of its part of its slice.
// kCoherent: the partial sums were written by this same launch (by other dies' workgroups, with write-through stores): they
// are read with loads that do not hit a line another die may have changed (byte offsets then fit 31 bits: host check).
template <int NW, int V, bool kCoherent = false>
__device__ __forceinline__ void finish_columns(const FinishArgs& a, const int block, const int nblocks, FinishShared<NW>& sh,
                                               const int predicted_raw, const bool any_wide = false) {
  const __amdgpu_buffer_rsrc_t rpart =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(a.partial), 0, kCoherent ? static_cast<int>(a.slice_stride * a.splits * 4) : 0, 0x00020000);
  constexpr int kSc1 = 16;   // cache policy bit: coherent across the dies' L2 caches
  const int units = static_cast<int>(a.nv);   // kCoherent: a column is a unit (four output channels), not four input channels
  // kMixed = false: no workgroup wrote a third plane, every sum is the sign-extended 24-bit value
  auto slice_col = [&](auto mixed, int z, long long col) -> v4i {
    if constexpr (kCoherent) {
      const int zoff = __builtin_amdgcn_readfirstlane(static_cast<int>(z * a.slice_stride * 4));   // z is the same in all lanes
      const v2u lo = __builtin_amdgcn_raw_buffer_load_b64(rpart, static_cast<int>(col) * 8, zoff, kSc1);
      const uint32_t mid = __builtin_amdgcn_raw_buffer_load_b32(rpart, units * 8 + static_cast<int>(col) * 4, zoff, kSc1);
      v4i r;   // biased sums, 24 bits each
      r[0] = static_cast<int>(__builtin_amdgcn_perm(mid, lo[0], 0x0C040100u));   // 0, mid.b0, lo.b1, lo.b0
      r[1] = static_cast<int>(__builtin_amdgcn_perm(mid, lo[0], 0x0C050302u));
      r[2] = static_cast<int>(__builtin_amdgcn_perm(mid, lo[1], 0x0C060100u));
      r[3] = static_cast<int>(__builtin_amdgcn_perm(mid, lo[1], 0x0C070302u));
      if constexpr (decltype(mixed)::value) {   // rare: the writer of this column's tile in slice z tells whether it wrote top bytes
        const uint32_t rt = static_cast<uint32_t>(col) / static_cast<uint32_t>(a.C);   // kg * 9 + t
        const uint32_t tile = (rt / 9u >> 5) + static_cast<uint32_t>(a.tiles_k) * ((static_cast<uint32_t>(col) - rt * static_cast<uint32_t>(a.C)) >> 5);
        const bool wide = __hip_atomic_load(a.wide + tile + static_cast<uint32_t>(a.tiles_k * a.tiles_c) * static_cast<uint32_t>(z), __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT) != 0u;
        uint32_t hi = 0;
        if (wide) hi = __builtin_amdgcn_raw_buffer_load_b32(rpart, units * 12 + static_cast<int>(col) * 4, zoff, kSc1);
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = static_cast<int>(static_cast<uint32_t>(r[e]) | ((hi >> (8 * e)) << 24));
      }
      return r;
    } else {
      return reinterpret_cast<const v4i*>(a.partial + z * a.slice_stride)[col];
    }
  };
  constexpr int OWN = V / NW > 0 ? V / NW : 1;   // columns a wavefront completes
  constexpr int VS = V < NW ? V : NW;            // columns a workgroup has when the slices are shared (fewer rounds than wavefronts)
  auto& part = sh.part;
  auto& wmax = sh.wmax;
  uint32_t& gshare = sh.gshare;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool has_prediction = a.predict != 0 && a.shift_out != nullptr;
  const bool trunc = a.trunc != 0;
  const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
  const bool same_layout = a.Cw == a.C;
  const uint32_t C = static_cast<uint32_t>(a.C), Cw = static_cast<uint32_t>(a.Cw);
  // division by the channel count: a shift for the usual powers of two (a 32-bit division is some forty instructions,
  // and this part of the launch runs few wavefronts)
  const int c_log2 = (C & (C - 1u)) == 0u ? 31 - __builtin_clz(C) : -1;
  auto div_c = [&](uint32_t x) -> uint32_t { return c_log2 >= 0 ? x >> c_log2 : x / C; };
  auto out_col = [&](long long col) -> long long {
    if constexpr (kCoherent) {
      const uint32_t rt = div_c(static_cast<uint32_t>(col)), c = static_cast<uint32_t>(col) - rt * C, kg = rt / 9u, tap = rt - kg * 9u;
      return static_cast<long long>(((kg * 4u + (c & 3u)) * 9u + tap) * (C >> 2) + (c >> 2));
    } else {
      return col;
    }
  };
  // the old weights are requested first: they depend on nothing and are wanted right after the sums
  uint32_t wold[OWN];
#pragma unroll
  for (int j = 0; j < OWN; ++j) {
    const int v = j * NW + wave;
    const long long col = (static_cast<long long>(v) * nblocks + block) * 64 + lane;
    wold[j] = (same_layout && v < V && col < a.nv) ? reinterpret_cast<const uint32_t*>(a.w)[out_col(col)] : 0u;
  }
  v4i fin[OWN];
  uint32_t lmax = 0;
  // Every wavefront has columns of its own at least in the first round (uniform over the grid): then each adds all
  // slices of its own columns and nothing goes through LDS.  With fewer columns than wavefronts the slices are
  // shared instead (phases 1 and 2 below), so that no wavefront idles while another walks over all slices.
  const bool direct = a.nv >= static_cast<long long>(NW) * nblocks * 64;
  // the whole gathering phase exists twice, so that the usual case (no third plane anywhere) has no branch between
  // its loads and keeps them all in flight
  const int bias_total = kCoherent ? static_cast<int>(static_cast<uint32_t>(a.splits) * kPartialBias) : 0;   // modulo 2^32, as the sums
  auto gather = [&](auto mixed) {
  if (direct) {
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int v = j * NW + wave;
      const long long col = (static_cast<long long>(v) * nblocks + block) * 64 + lane;
      v4i s = {0, 0, 0, 0};
      if (v < V && col < a.nv) {
        int z = 0;
        for (; z + 3 < a.splits; z += 4) {
          const v4i v0 = slice_col(mixed, z + 0, col);
          const v4i v1 = slice_col(mixed, z + 1, col);
          const v4i v2 = slice_col(mixed, z + 2, col);
          const v4i v3 = slice_col(mixed, z + 3, col);
          s += (v0 + v1) + (v2 + v3);
        }
        for (; z < a.splits; ++z) s += slice_col(mixed, z, col);
        s -= bias_total;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (a.roundtrip) s[e] = f32_roundtrip(s[e]);
        const uint32_t u = uabs(s[e]);
        lmax = u > lmax ? u : lmax;
      }
      fin[j] = s;
    }
  } else {
  v4i sum[VS];
  // phase 1: every wavefront adds its share of the slices for all of the workgroup's columns
#pragma unroll
  for (int v = 0; v < VS; ++v) {
    const long long col = (static_cast<long long>(v) * nblocks + block) * 64 + lane;
    v4i s = {0, 0, 0, 0};
    if (col < a.nv) {
      int z = wave;
      for (; z + 3 * NW < a.splits; z += 4 * NW) {
        const v4i v0 = slice_col(mixed, z + 0 * NW, col);
        const v4i v1 = slice_col(mixed, z + 1 * NW, col);
        const v4i v2 = slice_col(mixed, z + 2 * NW, col);
        const v4i v3 = slice_col(mixed, z + 3 * NW, col);
        s += (v0 + v1) + (v2 + v3);
      }
      for (; z < a.splits; z += NW) s += slice_col(mixed, z, col);
    }
    sum[v] = s;
  }
  // phase 2: column v is completed by wavefront v % NW (two LDS buffers in turn: one barrier per column)
#pragma unroll
  for (int v = 0; v < VS; ++v) {
    if (static_cast<long long>(v) * nblocks * 64 >= a.nv) continue;  // uniform over the grid: nothing at this stride
    part[v & 1][wave][lane] = sum[v];
    __syncthreads();
    if (wave == v % NW) {
      v4i s = part[v & 1][0][lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) s += part[v & 1][w][lane];
      if ((static_cast<long long>(v) * nblocks + block) * 64 + lane < a.nv) s -= bias_total;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (a.roundtrip) s[e] = f32_roundtrip(s[e]);
        const uint32_t u = uabs(s[e]);
        lmax = u > lmax ? u : lmax;
      }
      fin[v / NW] = s;
    }
  }
  }
  };
  if (kCoherent && any_wide) gather(std::true_type{});
  else gather(std::false_type{});
  // kCoherent: a lane holds four output channels of one input channel, its quad four consecutive input channels: a
  // 4 x 4 transposition inside the quad (two rounds of swaps) gives every lane four input channels of one output
  // channel, the form of the weights in memory, and out_col the column that is (quads lie inside one row: C % 4 == 0)
  if constexpr (kCoherent) {
    const bool odd1 = (lane & 1) != 0, odd2 = (lane & 2) != 0;
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      v4i s = fin[j], x;
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = __builtin_amdgcn_mov_dpp(s[e ^ 1], 0xB1, 0xf, 0xf, true);   // quad_perm:[1,0,3,2]
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] = (((e & 1) != 0) == odd1) ? s[e] : x[e];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = __builtin_amdgcn_mov_dpp(s[e ^ 2], 0x4E, 0xf, 0xf, true);   // quad_perm:[2,3,0,1]
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] = (((e & 2) != 0) == odd2) ? s[e] : x[e];
      fin[j] = s;
    }
  }
  lmax = wave_max_u32(lmax);
  if (lane == 0) wmax[wave] = lmax;
  __syncthreads();
  uint32_t bmax = 0;   // the workgroup's largest magnitude, in every wavefront
#pragma unroll
  for (int w = 0; w < NW; ++w) bmax = max(bmax, wmax[w]);
  if (wave == 0 && lane == 0)
    __hip_atomic_store(slot_word(a.sync + kFinishSlot0, block), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // phase 3: every wavefront rounds its columns and updates their weights (element counts fit 31 bits: host check).
  // With a predicted shift (a.predict) the update is applied before the range is final, so that its stores overlap
  // the wait for the other workgroups, and applied once more from the same old weights if the final shift differs.
  // shift: the same in every lane, but it has come through LDS or memory, which the compiler cannot know - as a scalar
  // the choices below are scalar branches instead of both sides under execution masks
  auto apply = [&](int shift_any, bool first) {
    const int shift = __builtin_amdgcn_readfirstlane(shift_any);
#pragma unroll
    for (int j = 0; j < OWN; ++j) {
      const int v = j * NW + wave;
      if (v >= V) continue;
      const long long gcol = (static_cast<long long>(v) * nblocks + block) * 64 + lane;
      if (gcol >= a.nv) continue;
      const long long col = out_col(gcol);
      const v4i s = fin[j];
      if (first && a.dw != nullptr) reinterpret_cast<v4i*>(a.dw)[col] = s;
      int r[4];
      if (shift < 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = wrap_to_i8(s[e]);
      } else if (psto) {
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(s[e], shift, trunc);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = round_one32<NITI_ROUND_NEAREST>(s[e], shift, trunc);
      }
      const uint32_t e0 = static_cast<uint32_t>(col) * 4u;
      const uint32_t rt = div_c(e0);            // k * 9 + tap
      const uint32_t c0 = e0 - rt * C;
      uint32_t wnew = 0;   // the four updated weights (zero where the gradient column is channel padding)
      if (same_layout) {
        uint32_t gp = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int wo = static_cast<int>(static_cast<int8_t>((wold[j] >> (8 * e)) & 0xFFu));
          wnew |= (static_cast<uint32_t>(clip127(wo - r[e])) & 0xFFu) << (8 * e);
          gp |= (static_cast<uint32_t>(r[e]) & 0xFFu) << (8 * e);
        }
        reinterpret_cast<uint32_t*>(a.w)[col] = wnew;
        if (a.g8 != nullptr) reinterpret_cast<uint32_t*>(a.g8)[col] = gp;
      } else {   // applied once only (the old weights are read here)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (c0 + e < Cw) {
            const uint32_t wi = rt * Cw + c0 + e;
            const int wn = clip127(static_cast<int>(a.w[wi]) - r[e]);
            a.w[wi] = static_cast<int8_t>(wn);
            wnew |= (static_cast<uint32_t>(wn) & 0xFFu) << (8 * e);
            if (a.g8 != nullptr) a.g8[wi] = static_cast<int8_t>(r[e]);
          }
        }
      }
      if (a.wprep != nullptr) {
        // [64-channel group][32-channel slice][tap][64 rows][32 bytes], 16-byte halves swapped where (row >> 3) is odd
        const uint32_t k = rt / 9u, tap = rt - k * 9u;
        const uint32_t row = k & 63u, cs = c0 >> 5;
        const uint32_t half = ((c0 >> 4) & 1u) ^ ((row >> 3) & 1u);
        const uint32_t dst = (((((k >> 6) * ((C + 31u) >> 5) + cs) * 9u + tap) * 64u + row) << 5) + half * 16u + (c0 & 15u);
        *reinterpret_cast<uint32_t*>(a.wprep + dst) = wnew;
      }
    }
  };
  const bool speculate = a.predict != 0 && same_layout && nblocks > 1;
  int applied = -1;
  if (speculate) {
    applied = max(max(bitwidth_of(bmax, a.bw_mode) - a.target_bits, 0), has_prediction ? predicted_raw : 0);
    apply(applied, true);
  }
  if (wave == 0) {
    const uint32_t g = wait_slots(a.sync + kFinishSlot0, nblocks, a.spin_limit, &a.sync[1], a.sticky);
    if (lane == 0) gshare = g != 0u ? g - 1u : 0u;
  }
  __syncthreads();
  const uint32_t gmax = gshare;
  const int shift = max(bitwidth_of(gmax, a.bw_mode) - a.target_bits, 0);
  if (block == 0 && threadIdx.x == 0) {
    a.sync[0] = gmax;
    if (a.shift_out != nullptr) *a.shift_out = shift;
    if (a.exp_out != nullptr)
      *a.exp_out = shift + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
  }
  if (shift != applied) {
    if (applied >= 0) __builtin_amdgcn_s_waitcnt(0);   // the first update's stores leave before those that replace them
    apply(shift, applied < 0);
  }
}

// ---- the same computation with half the partial-sum traffic ------------------------------------------------
// The kernel above leaves 128 x 64 x 9 partial sums (295 KB) per workgroup in memory; with about one workgroup
// per compute unit that is almost 60 MB per launch, written and read again, whatever the layer - more time than
// the matrix work.  Here a workgroup owns 128 x 32 x 9 sums: its 8 wavefronts are 4 output-channel quarters x 2
// pixel halves, the two halves are added through LDS at the end, and 147 KB per workgroup go to memory.  The
// error tile keeps its full 128-byte rows; the activation tile narrows to 32-byte slots (no swizzle needed: 8
// pixels x 16 channels read by 16 lanes cover 32 distinct banks, the other 16 lanes the other 32).  A stage is
// 256 output pixels.
template <int Q, int BR, int NI>
struct NGeom {
  static constexpr int RP = Q + 2;
  static constexpr int HR = BR + 2;
  static constexpr int SLOTS = NI * HR * RP;
  static constexpr int ACT_INSTR = (SLOTS + 31) / 32;       // an instruction fills 32 slots of 32 bytes
  static constexpr int ACT_BYTES = ACT_INSTR * 1024;
  static constexpr int ACT_LOADS = (ACT_INSTR + 7) / 8;
  static constexpr int ERR_BYTES = 256 * 128;               // 32 instructions of 8 pixels x 128 bytes
  static constexpr int STAGE_BYTES = ERR_BYTES + ACT_BYTES;
  static constexpr int STAGES = Q == 2 ? 2 : 3;             // the 2 x 2 maps' halo tile is as large as the error tile
  static constexpr int NL = 4 + ACT_LOADS;                  // loads per wavefront per stage
  static constexpr int REDUCE_BYTES = 4 * 9 * 16 * 64 * 4;  // four wavefronts park their accumulators
  static constexpr int LDS_BYTES = (STAGES * STAGE_BYTES > REDUCE_BYTES ? STAGES * STAGE_BYTES : REDUCE_BYTES) + 1024;
  static constexpr int HALF_ROWS = NI > 1 ? (NI / 2) * HR : 128 / Q;  // halo rows between the two pixel halves of a stage
  static constexpr int QUARTER_ROWS = NI > 1 ? (NI / 4) * HR : 64 / Q;  // ... between its four pixel quarters (kHalfK)
  static_assert(BR * NI * Q == 256, "a stage is 256 output pixels");
  static_assert(NI == 1 || BR == Q, "several images per stage only as whole images");
  static_assert(LDS_BYTES <= 160 * 1024, "stages must fit in LDS");
};

// kHalfK (at most 64 output channels): the wavefronts are 2 channel quarters x 4 pixel quarters instead of 4 x 2, so
// that none multiplies channels that do not exist.
template <int Q, int BR, int NI, bool kFinish, bool kHalfK>
__global__ __launch_bounds__(512, 1) void wgrad3x3_narrow_kernel(const WgradArgs a, const FinishArgs f) {
  using G = NGeom<Q, BR, NI>;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const dump = smem + G::LDS_BYTES - 1024;
  int predicted_raw = 0;
  if constexpr (kFinish) {
    // read at kernel start, looked at in the finishing part (see wgrad_finish_kernel)
    const bool has_prediction = f.predict != 0 && f.shift_out != nullptr;
    predicted_raw = __hip_atomic_load((has_prediction ? f.shift_out : reinterpret_cast<const int32_t*>(f.sync)) + opaque_zero(),
                                      __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const WorkItem item = die_local_work_item();
  const int k0 = item.x * 128;
  const int c0 = item.y * 32;
  const int band_begin = item.z * a.bands_per_split;   // bands of 256 pixels here
  const int band_end = min(band_begin + a.bands_per_split, a.bands);
  const int nb = band_end - band_begin;

  const __amdgpu_buffer_rsrc_t ract = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.act), 0, a.act_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rerr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.err), 0, a.err_bytes, 0x00020000);

  // ---- staging.  Error tile: an instruction fills 8 pixels x 128 bytes; lane -> (pixel lane/8, piece lane%8)
  int err_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int pix = (wave + 8 * i) * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((pix >> 1) & 7);
    const int ch = k0 + piece * 16;
    err_off[i] = ch < a.K ? pix * a.K + ch : kOob;
  }
  // Activation tile: NI images x HR rows x RP slots x 32 bytes, slots in a row; lane -> (slot lane/2, half lane%2)
  int act_off[G::ACT_LOADS];   // relative to image n0, row p0 = 0
  int act_hrow[G::ACT_LOADS];  // halo row, image index above bit 10
#pragma unroll
  for (int i = 0; i < G::ACT_LOADS; ++i) {
    const int slot = (wave + 8 * i) * 32 + (lane >> 1);
    const int row = slot / G::RP, col = slot - row * G::RP;
    const int ni = row / G::HR, h = row - ni * G::HR;
    const int ch = c0 + (lane & 1) * 16;
    const int iw = col - 1;
    int off = kOob;
    if (slot < G::SLOTS && iw >= 0 && iw < Q && ch < a.C) off = ((ni * Q + (h - 1)) * Q + iw) * a.C + ch;
    act_off[i] = off;
    act_hrow[i] = h + ni * 1024;
  }
  auto issue = [&](int band, int st) {
    int8_t* base = smem + st * G::STAGE_BYTES;
    const int pixbase = band * 256;
    const int n0 = pixbase / (Q * Q);
    const int p0 = (pixbase - n0 * (Q * Q)) / Q;
    const int eb = pixbase * a.K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = err_off[i] == kOob ? kOob : eb + err_off[i];
      int8_t* dst = base + (wave + 8 * i) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rerr, NITI_LDS(dst), 16, off, 0, 0, 0);
    }
    const int ab = (n0 * Q + p0) * Q * a.C;
#pragma unroll
    for (int i = 0; i < G::ACT_LOADS; ++i) {
      const int idx = wave + 8 * i;
      const int ih = p0 + (act_hrow[i] & 1023) - 1;
      const bool ok = act_off[i] != kOob && ih >= 0 && ih < Q && n0 + (act_hrow[i] >> 10) < a.N;
      const int off = ok ? ab + act_off[i] : kOob;
      int8_t* dst = idx < G::ACT_INSTR ? base + G::ERR_BYTES + idx * 1024 : dump;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ract, NITI_LDS(dst), 16, off, 0, 0, 0);
    }
  };

  // ---- fragment addressing (transposing LDS reads, see the kernel above)
  const int j = lane & 15;
  const int gg = (lane >> 4) & 1;
  const int lk = lane >> 5;
  const int wk = kHalfK ? wave & 1 : wave & 3;     // 32-output-channel quarter of the tile
  const int ph = kHalfK ? wave >> 1 : wave >> 2;   // 128-pixel half (64-pixel quarter) of a stage
  constexpr int kWavePixels = kHalfK ? 64 : 128;
  constexpr int kPartRows = kHalfK ? G::QUARTER_ROWS : G::HALF_ROWS;
  static_assert(!kHalfK || Q >= 8, "pixel quarters only for rows of at least 8 pixels");
  int a_base[2];
  // Rows of at least 8 pixels: the second and third tap of a filter row are byte shifts of the first one's pixels
  // (3 or 4 reads per filter row).  Shorter rows (4 x 4 and 2 x 2 maps: eight pixels are two or four rows) read
  // every tap.
  constexpr bool kShiftTaps = Q >= 8;
  constexpr bool kShiftErr = Q == 8 || Q == 16;   // the error fragment is shifted instead, once for all three filter rows
  constexpr int NB = kShiftErr ? 2 : (kShiftTaps ? (Q >= 16 ? 3 : 4) : 6);
  int b_base[NB];
#pragma unroll
  for (int o = 0; o < 2; ++o) {
    const int lpix = 16 * lk + 8 * o + (j >> 1);
    const int cb = wk * 32 + gg * 16 + 8 * (j & 1);
    a_base[o] = (ph * kWavePixels + lpix) * 128 + ((((cb >> 4) ^ ((lpix >> 1) & 7)) << 4) | (cb & 15));
  }
  {
    const int cb = gg * 16 + 8 * (j & 1);
    // lrow: output row inside the 32 pixels of a reduction step (which may span several whole images)
    auto slot_addr = [&](int lrow, int w) {
      const int hrow = (lrow / BR) * G::HR + lrow % BR;
      return G::ERR_BYTES + ((ph * kPartRows + hrow) * G::RP + w) * 32 + cb;
    };
    const int p0 = 16 * lk + (j >> 1), p1 = p0 + 8;
    if constexpr (kShiftErr) {
      b_base[0] = slot_addr(p0 / Q, p0 % Q + 1);
      b_base[1] = slot_addr(p1 / Q, p1 % Q + 1);
    } else if (!kShiftTaps) {
#pragma unroll
      for (int t = 0; t < 3; ++t) {
        b_base[2 * t] = slot_addr(p0 / Q, p0 % Q + t);
        b_base[2 * t + 1] = slot_addr(p1 / Q, p1 % Q + t);
      }
    } else if (Q >= 16) {
      b_base[0] = slot_addr(p0 / Q, p0 % Q);
      b_base[1] = slot_addr(p1 / Q, p1 % Q);
      b_base[2] = slot_addr(p0 / Q, p0 % Q + 16);
    } else {
      b_base[0] = slot_addr(p0 / Q, p0 % Q);
      b_base[1] = slot_addr(p0 / Q, p0 % Q + 8);
      b_base[2] = slot_addr(p1 / Q, p1 % Q);
      b_base[NB - 1] = slot_addr(p1 / Q, p1 % Q + 8);
    }
  }

  v16i acc[9];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[t][e] = 0;

#pragma unroll
  for (int s = 0; s < G::STAGES - 1; ++s)
    if (s < nb) issue(band_begin + s, s);

  for (int it = 0; it < nb; ++it) {
    if (it + G::STAGES - 2 < nb) wg_wait_vmcnt<(G::STAGES - 2) * G::NL>();
    else wg_wait_vmcnt<0>();
    wg_sync();
    wgrad_stage<Q, BR, G::HR, G::RP * 32, kShiftTaps, NB, kShiftErr, kHalfK ? 2 : 4>(
        lds_addr(smem + (it % G::STAGES) * G::STAGE_BYTES), a_base, b_base, acc,
        [&] { if (it + G::STAGES - 1 < nb) issue(band_begin + it + G::STAGES - 1, (it + G::STAGES - 1) % G::STAGES); });
  }

  // ---- add the two pixel halves: half 1 -> LDS -> half 0 -> memory.  Slot layout [value][lane].
  __syncthreads();  // all tiles consumed, no load in flight (the last stage was waited for with vmcnt(0))
  int32_t* const park = reinterpret_cast<int32_t*>(smem) + wk * (9 * 16 * 64) + lane;
  if constexpr (kHalfK) {
    // four pixel quarters: 1 -> 0 and 3 -> 2 first (four parked wavefronts fill the area), then 2 -> 0 like the halves
    int32_t* const park2 = park + (ph >> 1) * (2 * 9 * 16 * 64);
    if ((ph & 1) != 0) {
#pragma unroll
      for (int t = 0; t < 9; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) park2[(t * 16 + e) * 64] = acc[t][e];
    }
    __syncthreads();
    if ((ph & 1) == 0) {
#pragma unroll
      for (int t = 0; t < 9; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] += park2[(t * 16 + e) * 64];
    }
    __syncthreads();
  }
  if (ph == (kHalfK ? 2 : 1)) {
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) park[(t * 16 + e) * 64] = acc[t][e];
  }
  __syncthreads();
  // partial sums: acc[t][4g+e] = dw[k0+wk*32+8g+4*lk+e][tap t][c0+(lane&31)]
  const int c = c0 + (lane & 31);
  if constexpr (!kFinish) {
    if (ph == 0) {
      int32_t* out = a.partial + static_cast<long long>(item.z) * a.slice_stride;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int k = k0 + wk * 32 + g * 8 + lk * 4 + e;
#pragma unroll
          for (int t = 0; t < 9; ++t) {
            const int v = acc[t][4 * g + e] + park[(t * 16 + 4 * g + e) * 64];
            if (c < a.Cp && k < a.K) out[(static_cast<long long>(k) * 9 + t) * a.Cp + c] = v;
          }
        }
    }
  } else {
    // ---- the finishing pass in the same launch: all workgroups are resident (the host checks), every one takes a
    // share of the gradient's columns once the partial sums of all of them are in memory.  The sums travel between
    // the dies by write-through stores, completed before the arrival slot is filled, and by loads that bypass stale
    // lines (fences would do the same by writing back and invalidating whole L2 caches, once per wavefront: 50 us).
    // What bounds this part is the bytes, so the sums go as 24-bit values whenever all of the workgroup's fit (planes
    // of 16 and 8 bits; a third plane with the top bytes only when they do not).
    // a lane holds four consecutive output channels of one (tap, input channel): one unit of each plane, and 32 lanes
    // (input channels) make every store instruction whole 128-byte lines.  The values go biased by 2^23, so that the
    // reader adds zero-extended 24-bit numbers and takes the bias off once per column.
    const __amdgpu_buffer_rsrc_t rout =
        __builtin_amdgcn_make_buffer_rsrc(a.partial, 0, static_cast<int>(a.slice_stride * f.splits * 4), 0x00020000);
    constexpr int kSc1 = 16;   // written through to memory
    const int zoff = static_cast<int>(item.z * a.slice_stride * 4);
    const int units = static_cast<int>(f.nv);
    uint32_t over = 0;   // bits above the 24 of any biased value
    if (ph == 0) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int k = k0 + wk * 32 + g * 8 + lk * 4;
        const bool live = c < a.Cp && k < a.K;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
          uint32_t v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = static_cast<uint32_t>(acc[t][4 * g + e] + park[(t * 16 + 4 * g + e) * 64]) + kPartialBias;
            acc[t][4 * g + e] = static_cast<int>(v[e]);
            over |= v[e];
          }
          const int u = ((k >> 2) * 9 + t) * a.Cp + c;
          v2u lo;
          lo[0] = __builtin_amdgcn_perm(v[1], v[0], 0x05040100u);   // v1.b1 v1.b0 v0.b1 v0.b0
          lo[1] = __builtin_amdgcn_perm(v[3], v[2], 0x05040100u);
          const uint32_t m01 = __builtin_amdgcn_perm(v[1], v[0], 0x0C0C0602u);   // 0 0 v1.b2 v0.b2
          const uint32_t m23 = __builtin_amdgcn_perm(v[3], v[2], 0x06020C0Cu);   // v3.b2 v2.b2 0 0
          __builtin_amdgcn_raw_buffer_store_b64(lo, rout, live ? u * 8 : kOob, zoff, kSc1);
          __builtin_amdgcn_raw_buffer_store_b32(m01 | m23, rout, live ? units * 8 + u * 4 : kOob, zoff, kSc1);
        }
      }
    }
    // does any value of the workgroup need the third plane
    over = __builtin_amdgcn_readfirstlane(static_cast<int>(wave_max_u32(over >> 24)));
    uint32_t* const wgm = reinterpret_cast<uint32_t*>(dump);   // no load is in flight any more
    if (lane == 0) wgm[wave] = over;
    __syncthreads();
    uint32_t m = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) m |= wgm[w];
    const bool wide = __builtin_amdgcn_readfirstlane(static_cast<int>(m)) != 0;
    if (wide && ph == 0) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int k = k0 + wk * 32 + g * 8 + lk * 4;
        const bool live = c < a.Cp && k < a.K;
#pragma unroll
        for (int t = 0; t < 9; ++t) {
          const uint32_t v0 = acc[t][4 * g], v1 = acc[t][4 * g + 1], v2 = acc[t][4 * g + 2], v3 = acc[t][4 * g + 3];
          const uint32_t h01 = __builtin_amdgcn_perm(v1, v0, 0x0C0C0703u), h23 = __builtin_amdgcn_perm(v3, v2, 0x07030C0Cu);
          const int u = ((k >> 2) * 9 + t) * a.Cp + c;
          __builtin_amdgcn_raw_buffer_store_b32(h01 | h23, rout, live ? units * 12 + u * 4 : kOob, zoff, kSc1);
        }
      }
    }
    const int nblocks = static_cast<int>(gridDim.x * gridDim.y * gridDim.z);
    const int block = static_cast<int>(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's stores have been performed
    __syncthreads();
    if (tid == 0) {
      if (wide) {
        __hip_atomic_store(f.wide + item.x + f.tiles_k * (item.y + f.tiles_c * item.z), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(0x0F70);
      }
      // the slot's value also says which form this workgroup used: the largest over all slots tells every workgroup
      // whether it has to look at the per-workgroup words at all
      __hip_atomic_store(slot_word(f.arrive, block), wide ? 2u : 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (wave == 0) {
      const uint32_t seen = wait_slots(f.arrive, nblocks, f.spin_limit, &f.sync[1], f.sticky, 2u);
      if (lane == 0) wgm[8] = seen;
    }
    __syncthreads();
    const bool any_wide = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(wgm[8]))) >= 2u;
    finish_columns<8, kFusedV, true>(f, block, nblocks, *reinterpret_cast<FinishShared<8>*>(smem), predicted_raw, any_wide);
  }
}

// dw[e] = sum_z partial[z][e]; optional fp32 round trip; max |dw| folded into *absmax.
// A workgroup owns 64 int4 columns; its 4 wavefronts each add every 4th slice, then combine in LDS.
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const int32_t* __restrict__ partial, int32_t* __restrict__ dw,
                                                           int64_t nelem, int64_t n, int splits, int roundtrip,
                                                           uint32_t* absmax) {
  __shared__ v4i part[3][64];
  const int64_t nv = nelem >> 2;  // n below is the slice stride
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t col = static_cast<int64_t>(blockIdx.x) * 64 + lane;
  v4i s = {0, 0, 0, 0};
  if (col < nv) {
    int z = wave;
    for (; z + 12 < splits; z += 16) {
      const v4i v0 = reinterpret_cast<const v4i*>(partial + (z + 0) * n)[col];
      const v4i v1 = reinterpret_cast<const v4i*>(partial + (z + 4) * n)[col];
      const v4i v2 = reinterpret_cast<const v4i*>(partial + (z + 8) * n)[col];
      const v4i v3 = reinterpret_cast<const v4i*>(partial + (z + 12) * n)[col];
      s += (v0 + v1) + (v2 + v3);
    }
    for (; z < splits; z += 4) s += reinterpret_cast<const v4i*>(partial + z * n)[col];
  }
  if (wave > 0) part[wave - 1][lane] = s;
  __syncthreads();
  uint32_t lmax = 0;
  if (wave == 0 && col < nv) {
    s += part[0][lane] + part[1][lane] + part[2][lane];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (roundtrip) s[e] = f32_roundtrip(s[e]);
      const uint32_t u = uabs(s[e]);
      lmax = u > lmax ? u : lmax;
    }
    reinterpret_cast<v4i*>(dw)[col] = s;
  }
  if (absmax != nullptr && wave == 0) fold_absmax(absmax, lmax);
}

template <int NW>
__global__ __launch_bounds__(NW * 64, 4) void wgrad_finish_kernel(const FinishArgs a) {
  __shared__ FinishShared<NW> sh;
  // Read before this workgroup fills its slot: workgroup 0 overwrites the word only after all slots are filled.
  // An unconditional load (from the range word when there is no prediction) with an address that looks lane-dependent
  // to the compiler, whose result is first looked at after the partial sums have been added: a load inside a branch, or
  // one whose result is known to be uniform, would be waited for on the spot, in front of theirs.
  const bool has_prediction = a.predict != 0 && a.shift_out != nullptr;
  const int predicted_raw = __hip_atomic_load((has_prediction ? a.shift_out : reinterpret_cast<const int32_t*>(a.sync)) + opaque_zero(),
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  finish_columns<NW, kFinishV>(a, static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x), sh, predicted_raw);
}

// Slices are spaced so that the same element of consecutive slices falls into different memory
// channels (a stride that is a multiple of 64 KB would put them all into one).
long long slice_stride_for(int C, int K) {
  const long long n = static_cast<long long>(K) * 9 * C;
  return (n + 1023) / 1024 * 1024 + 1088;
}

// The narrow-tile arrangement needs whole stages of 256 pixels.  NITI_WGRAD_NARROW=0/1 pins the choice (tests).
bool use_narrow_arrangement(int N, int Q) {
  const bool fits = (static_cast<long long>(N) * Q * Q) % 256 == 0;
  if (Q < 8) return true;   // the only arrangement for the small maps (the shape check requires whole stages)
  const char* e = getenv("NITI_WGRAD_NARROW");
  if (e != nullptr) return e[0] == '1' && fits;
  return fits;
}

int pick_splits(int N, int Q, int C, int K) {
  const char* e = getenv("NITI_WGRAD_BLOCKS");
  int target = e != nullptr ? atoi(e) : 0;
  int bands, tiles;
  if (use_narrow_arrangement(N, Q)) {
    bands = N * Q * Q / 256;
    tiles = ((K + 127) / 128) * ((C + 31) / 32);
    if (target < 1) target = 256;
  } else {
    bands = N * Q * Q / 128;
    tiles = ((K + 127) / 128) * ((C + 63) / 64);
    if (target < 1) target = 192;  // fewer, longer workgroups: less partial-sum traffic per MFMA
  }
  int splits = (target + tiles - 1) / tiles;
  if (splits > bands) splits = bands;
  if (splits < 1) splits = 1;
  const int per = (bands + splits - 1) / splits;
  return (bands + per - 1) / per;
}

// f != nullptr: the one-launch form (main loop + finishing pass); returns NITI_ERR_UNSUPPORTED without launching when its
// grid would not be resident at once, and the caller then runs the pair of launches.
template <int Q, int BR, int NI, bool kFinish, bool kHalfK>
int launch_narrow_geom_as(const WgradArgs& a, int splits, hipStream_t stream, const FinishArgs& f) {
  using G = NGeom<Q, BR, NI>;
  constexpr size_t lds = G::LDS_BYTES;
  auto k = wgrad3x3_narrow_kernel<Q, BR, NI, kFinish, kHalfK>;
  static bool attr_set_of[kDeviceSlots] = {};   // function attributes are per device
  static int resident_of[kDeviceSlots] = {};    // workgroups of this kernel the device holds at once
  bool& attr_set = attr_set_of[device_slot()];
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "wgrad: cannot reserve %zu bytes of LDS", lds);
    if (kFinish) {
      int dev = 0, cus = 0, per = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
          hipOccupancyMaxActiveBlocksPerMultiprocessor(&per, reinterpret_cast<const void*>(k), 512, lds) != hipSuccess)
        return fail(NITI_ERR_LAUNCH, "wgrad: cannot query occupancy");
      resident_of[device_slot()] = cus * per;
    }
    attr_set = true;
  }
  dim3 grid((a.K + 127) / 128, (a.C + 31) / 32, splits);
  if (kFinish) {
    const long long nblocks = static_cast<long long>(grid.x) * grid.y * grid.z;
    if (nblocks > resident_of[device_slot()] || nblocks > kArriveSlots || f.nv > nblocks * kFusedV * 64 ||
        f.slice_stride * f.splits * 4 >= 0x7fffffffLL)
      return NITI_ERR_UNSUPPORTED;
  }
  hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, a, f);
  return check_launch("wgrad3x3_narrow");
}

template <int Q, int BR, int NI>
int launch_narrow_geom(const WgradArgs& a, int splits, hipStream_t stream, const FinishArgs* f) {
  if constexpr (Q >= 8) {
    const bool half_k = a.K <= 64;   // two channel quarters x four pixel quarters
    if (f != nullptr)
      return half_k ? launch_narrow_geom_as<Q, BR, NI, true, true>(a, splits, stream, *f) : launch_narrow_geom_as<Q, BR, NI, true, false>(a, splits, stream, *f);
    return half_k ? launch_narrow_geom_as<Q, BR, NI, false, true>(a, splits, stream, FinishArgs{})
                  : launch_narrow_geom_as<Q, BR, NI, false, false>(a, splits, stream, FinishArgs{});
  } else {
    if (f != nullptr) return NITI_ERR_UNSUPPORTED;
    return launch_narrow_geom_as<Q, BR, NI, false, false>(a, splits, stream, FinishArgs{});
  }
}

template <int Q, int BR, int NI>
int launch_geom(const WgradArgs& a, int splits, hipStream_t stream) {
  using G = Geom<Q, BR, NI>;
  constexpr int STAGES = 3;
  constexpr size_t lds = static_cast<size_t>(STAGES) * G::STAGE_BYTES + 1024;
  static_assert(lds <= 160 * 1024, "stages must fit in LDS");
  auto k = wgrad3x3_kernel<Q, BR, NI, STAGES>;
  static bool attr_set_of[kDeviceSlots] = {};   // function attributes are per device
  bool& attr_set = attr_set_of[device_slot()];
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "wgrad: cannot reserve %zu bytes of LDS", lds);
    attr_set = true;
  }
  dim3 grid((a.K + 127) / 128, (a.C + 63) / 64, splits);
  hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, a);
  return check_launch("wgrad3x3");
}

}  // namespace

bool wgrad3x3_supported(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (R != 3 || S != 3 || stride != 1 || pad != 1 || H != W) return false;
  if (H != 2 && H != 4 && H != 8 && H != 16 && H != 32) return false;
  if (C % 16 != 0 || K % 16 != 0) return false;
  const long long pix = static_cast<long long>(N) * H * W;
  if (pix % 128 != 0) return false;  // bands of 128 pixels: whole rows / whole images
  if (H <= 4 && pix % 256 != 0) return false;  // small maps: only the arrangement with stages of 256 pixels
  if (H == 8 && N % 2 != 0) return false;
  if (pix * C >= 0x7fffffffLL || pix * K >= 0x7fffffffLL) return false;
  return true;
}

size_t wgrad3x3_workspace(int N, int H, int C, int K) {
  return static_cast<size_t>(pick_splits(N, H, C, K)) * slice_stride_for(C, K) * sizeof(int32_t);
}

static int launch_wgrad3x3_partials(const int8_t* act, const int8_t* err, int N, int H, int C, int K, int Cp, void* workspace,
                                    WgradArgs& a, int& splits, hipStream_t stream, FinishArgs* finish = nullptr) {
  a.act = act;
  a.err = err;
  a.partial = static_cast<int32_t*>(workspace);
  a.slice_stride = slice_stride_for(Cp, K);
  a.N = N;
  a.C = C;
  a.K = K;
  a.Cp = Cp;
  const bool narrow = use_narrow_arrangement(N, H);
  a.bands = N * H * H / (narrow ? 256 : 128);
  splits = pick_splits(N, H, C, K);
  a.bands_per_split = (a.bands + splits - 1) / splits;
  a.act_bytes = static_cast<long long>(N) * H * H * C;
  a.err_bytes = static_cast<long long>(N) * H * H * K;
  if (finish != nullptr) {
    if (!narrow) return NITI_ERR_UNSUPPORTED;
    finish->partial = a.partial;
    finish->slice_stride = a.slice_stride;
    finish->splits = splits;
    finish->tiles_k = (K + 127) / 128;
    finish->tiles_c = (C + 31) / 32;
  }
  if (narrow) {
    if (H == 32) return launch_narrow_geom<32, 8, 1>(a, splits, stream, finish);
    if (H == 16) return launch_narrow_geom<16, 16, 1>(a, splits, stream, finish);
    if (H == 8) return launch_narrow_geom<8, 8, 4>(a, splits, stream, finish);
    if (H == 4) return launch_narrow_geom<4, 4, 16>(a, splits, stream, finish);
    return launch_narrow_geom<2, 2, 64>(a, splits, stream, finish);
  }
  if (H == 32) return launch_geom<32, 4, 1>(a, splits, stream);
  if (H == 16) return launch_geom<16, 8, 1>(a, splits, stream);
  return launch_geom<8, 8, 2>(a, splits, stream);
}

int launch_wgrad3x3(const int8_t* act, const int8_t* err, int32_t* dw, int N, int H, int C, int K, bool roundtrip,
                    uint32_t* absmax, void* workspace, hipStream_t stream) {
  WgradArgs a;
  int splits = 1;
  const int st = launch_wgrad3x3_partials(act, err, N, H, C, K, C, workspace, a, splits, stream);
  if (st != NITI_OK) return st;
  const int64_t n = static_cast<int64_t>(K) * 9 * C;
  int64_t g = (n / 4 + 63) / 64;
  if (g < 1) g = 1;
  hipLaunchKernelGGL(wgrad_reduce_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0, stream, a.partial, dw, n,
                     static_cast<int64_t>(a.slice_stride), splits, roundtrip ? 1 : 0, absmax);
  return check_launch("wgrad_reduce");
}

// Workgroups of the finishing kernel for a [K][9][C] gradient (= sync slots), or 0 when it is too large for
// the kernel's per-workgroup share.
int wgrad3x3_finish_blocks(int C, int K) {
  const long long groups = (static_cast<long long>(K) * 9 * C / 4 + 63) / 64;
  const long long nb = groups < 1024 ? groups : 1024;
  if (groups > nb * kFinishV) return 0;
  return static_cast<int>(nb < 1 ? 1 : nb);
}

// header, range slots (of the finishing launch or of the one-launch form, whichever has more workgroups), arrival slots
static size_t range_slot_words(int blocks) { return slot_words(blocks > kArriveSlots ? blocks : kArriveSlots); }
// ... and the words that say which workgroups wrote int32 sums (one-launch form)
size_t wgrad3x3_sync_words(int blocks) {
  return static_cast<size_t>(kFinishSlot0) + range_slot_words(blocks) + slot_words(kArriveSlots) + 16 + kArriveSlots;
}
static size_t wgrad3x3_arrive_offset(int C, int K) { return static_cast<size_t>(kFinishSlot0) + range_slot_words(wgrad3x3_finish_blocks(C, K)); }

int launch_wgrad3x3_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int H, int C, int K,
                           bool roundtrip, uint32_t* sync, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep,
                           void* workspace, hipStream_t stream) {
  // The first layer's three input channels come padded to 16: unless the caller wants the int32 gradient in that
  // layout, the partial sums keep four columns per tap (a quarter of the bytes written and read back).
  const int Cp = (dw == nullptr && C == 16 && w_channels <= 4) ? 4 : C;
  const int nb = wgrad3x3_finish_blocks(Cp, K);
  if (nb == 0) return fail(NITI_ERR_UNSUPPORTED, "wgrad_update: gradient of %d x 9 x %d too large for the single-pass finish", K, C);
  if (static_cast<long long>(K) * 9 * C >= 0x7fffffffLL) return fail(NITI_ERR_UNSUPPORTED, "wgrad_update: gradient of %d x 9 x %d too large", K, C);
  {
    // the first layer: one launch with integer atomics and a last-arriver finish (NITI_WGRAD_FIRST=0 pins the pair below)
    const char* e = getenv("NITI_WGRAD_FIRST");
    if ((e == nullptr || e[0] != '0') && wgrad_first_supported(N, H, C, K, w_channels)) {
      int32_t* const accum = reinterpret_cast<int32_t*>(sync + wgrad3x3_sync_words(wgrad3x3_finish_blocks(C, K)));
      return launch_wgrad_first_update(act, err, w, w_channels, N, K, roundtrip, sync, accum, rq, g8, dw, wprep, stream);
    }
  }
  {
    // few pixels, many weights: nothing to split, one launch does it all (NITI_WGRAD_SMALL=0 pins the kernel pair below)
    const char* e = getenv("NITI_WGRAD_SMALL");
    if ((e == nullptr || e[0] != '0') && wgrad_small_supported(N, H, C, K, w_channels))
      return launch_wgrad_small_update(act, err, w, N, H, C, K, roundtrip, sync, rq, g8, dw, wprep, stream);
  }
  if (!wgrad3x3_supported(N, H, H, C, K, 3, 3, 1, 1))
    return fail(NITI_ERR_UNSUPPORTED, "wgrad_update: %d pixels on %d x %d maps run only as the one-launch kernel, which this call cannot use", N * H * H, H, H);
  static int resident_of[kDeviceSlots][2] = {};   // workgroups of 4 / 16 wavefronts the device holds at once
  int* const resident = resident_of[device_slot()];
  if (resident[0] == 0) {
    int dev = 0, cus = 0, per4 = 0, per16 = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per4, reinterpret_cast<const void*>(wgrad_finish_kernel<4>), 256, 0) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per16, reinterpret_cast<const void*>(wgrad_finish_kernel<16>), 1024, 0) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "wgrad_update: cannot query occupancy");
    resident[0] = cus * per4;
    resident[1] = cus * per16;
  }
  if (nb > resident[0]) return fail(NITI_ERR_UNSUPPORTED, "wgrad_update: %d workgroups do not fit on the device at once (%d)", nb, resident[0]);
  WgradArgs a;
  int splits = 1;
  FinishArgs f{};
  f.nv = static_cast<long long>(K) * 9 * Cp / 4;
  f.C = Cp;
  f.Cw = w_channels;
  f.w = w;
  f.g8 = g8;
  f.dw = dw;
  f.wprep = wprep;
  f.sync = sync;
  f.roundtrip = roundtrip ? 1 : 0;
  f.target_bits = rq.target_bits;
  f.method = rq.method;
  f.trunc = rq.trunc;
  f.predict = (rq.flags & NITI_RQ_SHIFT_HINT) != 0 ? 1 : 0;
  f.bw_mode = rq.bw_mode;
  f.spin_limit = rq.spin_limit;
  f.sticky = rq.sticky;
  f.shift_out = rq.shift_out;
  f.exp_a = rq.exp_a;
  f.exp_b = rq.exp_b;
  f.exp_out = rq.exp_out;
  f.arrive = sync + wgrad3x3_arrive_offset(C, K);
  f.wide = f.arrive + slot_words(kArriveSlots);
  {
    // main loop and finishing pass as one launch where its grid is resident at once (NITI_WGRAD_ONE_LAUNCH=0 pins the pair)
    const char* e = getenv("NITI_WGRAD_ONE_LAUNCH");
    if (e == nullptr || e[0] != '0') {
      const int st1 = launch_wgrad3x3_partials(act, err, N, H, C, K, Cp, workspace, a, splits, stream, &f);
      if (st1 != NITI_ERR_UNSUPPORTED) return st1;
    }
  }
  const int st = launch_wgrad3x3_partials(act, err, N, H, C, K, Cp, workspace, a, splits, stream);
  if (st != NITI_OK) return st;
  f.partial = a.partial;
  f.slice_stride = a.slice_stride;
  f.splits = splits;
  // many slices and few columns per workgroup: sixteen wavefronts share the slices
  if (splits >= 32 && nb <= resident[1]) hipLaunchKernelGGL(wgrad_finish_kernel<16>, dim3(nb), dim3(1024), 0, stream, f);
  else hipLaunchKernelGGL(wgrad_finish_kernel<4>, dim3(nb), dim3(256), 0, stream, f);
  return check_launch("wgrad_finish");
}

}  // namespace niti
