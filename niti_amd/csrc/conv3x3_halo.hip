// int8 3x3 / stride 1 / pad 1 convolution forward on the gfx950 matrix cores with the activation
// halo tile resident in LDS ("read every activation once, not once per filter tap").
//
// The plain implicit GEMM (conv_mfma.hip) fetches each activation nine times and each filter row
// once per pixel tile through L2.  Here a workgroup owns 256 consecutive output pixels (whole rows of
// an image, or whole small images) x KT output channels (128; 64, or on small maps 32, when the launch would
// otherwise leave compute units idle) and walks over the input channels in slices of 32 - one reduction step of
// v_mfma_i32_32x32x32_i8.  Per slice it stages the activation rows with their one-pixel halo once
// (10-20 KB, out-of-image positions read as zero through an out-of-range buffer offset) and serves all
// nine taps from that tile; the filter streams one filter row (three taps) per stage from a
// pre-arranged copy whose memory image is exactly the swizzled LDS tile, so every load instruction
// moves contiguous bytes.
//
// 8 wavefronts: 4 pixel groups of 64 x 2 channel groups of KT/2; a wavefront holds 2 x KT/64 tiles of
// 32 x 32 sums (KT = 32: 8 pixel groups of 32, one tile each).  Activation slices are double buffered and the filter stages run through a ring of
// three, so the only synchronisation is one s_barrier per filter row; all of it stays under 80 KB of
// LDS and 128 VGPRs, so two workgroups share a compute unit and fill each other's stalls.  The same
// kernel computes the data gradient when given the flipped / transposed filter arrangement (prepare
// kernel, mode 1).
//
// Requantising variant (kFused): the int32 sums never leave the registers.  Every workgroup publishes
// the largest magnitude of its tile in a slot of its own, waits until the slots of all workgroups of the
// launch are filled (they are all resident - the host checks that - and the wait is bounded by a wall-clock
// limit so that every wavefront exits whatever happens), derives the tensor-wide shift from the maximum
// over the slots and stores rounded int8.  Compared with the int32 store + separate requantisation pass
// this removes 8 of the 9 bytes moved per output element.  The same epilogue can leave the 2x2 / stride-2
// maximum of its output next to it (the max-pool that follows the layer).
//
// Launches the device cannot hold at once: the 64-channel tile takes 512 pixels per workgroup where that
// is enough (HGeom::TWO); otherwise the launch runs twice without waiting (kRqNoWait, kRqSettle below).
// Maps of 2 x 2 pixels have a kernel of their own at the end of this file (conv3x3_map2_kernel).
#include <stdlib.h>

#include "common.h"
#include "lds_asm.h"
#include "requant_math.h"

namespace niti {
namespace {

constexpr int kOob = -1;
constexpr int kOobFar = static_cast<int>(0x80000000u);   // out of range whatever scalar offset below 2^31 is added

// s_waitcnt vmcnt(N) with the other counters left alone
template <int N>
__device__ inline void hc_wait_vmcnt() {
  static_assert(N >= 0 && N <= 15);
  __builtin_amdgcn_s_waitcnt(0x0F70 | N);
}
// the same for a wavefront that has N loads in flight if it issues the full number of filter loads per stage and
// N - 1 if it issues one fewer (the count is an immediate, so the choice is a branch on a wavefront-uniform flag)
template <int N>
__device__ inline void hc_wait_vmcnt_pair(bool full) {
  if (full)
    hc_wait_vmcnt<N>();
  else
    hc_wait_vmcnt<N - 1>();
}
__device__ inline void hc_sync() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// The four dwords of a fragment, each lane taking its right-hand neighbour's (kLeft: wave_shl:1) or its left-hand
// neighbour's (wave_shr:1) value - zero where there is none - and-ed with keep.  The shift rides on the AND as its DPP
// modifier: one instruction per dword where a DPP move followed by the AND would be two.  The compiler does not see
// inside the statement, so the wait states it would add are written out: two in front (a vector instruction that
// wrote a source just before), two behind (an MFMA that reads the result right after).
template <bool kLeft>
__device__ inline v4i shifted_and4(v4i x, int keep) {
  int r0, r1, r2, r3;
  if constexpr (kLeft)
    asm("s_nop 1\n\t"
        "v_and_b32_dpp %0, %4, %8 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %1, %5, %8 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %2, %6, %8 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %3, %7, %8 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "s_nop 1"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(keep));
  else
    asm("s_nop 1\n\t"
        "v_and_b32_dpp %0, %4, %8 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %1, %5, %8 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %2, %6, %8 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "v_and_b32_dpp %3, %7, %8 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
        "s_nop 1"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]), "v"(keep));
  return v4i{r0, r1, r2, r3};
}

struct HaloArgs {
  const int8_t* x;    // [N,Q,Q,C]
  const int8_t* wp;   // prepared filter: [ceil(K/64)][cslices][9][64][32], rows XOR-swizzled
  int32_t* y;         // [N,Q,Q,K]
  uint32_t* absmax;
  int N, C, K;
  int cslices;        // ceil(C / 32)
  int src_cslices;    // kWT only: 32-channel slices of the forward filter copy read as the data gradient's filter
  long long x_bytes, wp_bytes, y_bytes;
  unsigned flags;
  // requantising variant only
  int8_t* y8;         // [N,Q,Q,K] int8
  const int8_t* mask; // optional [N,Q,Q,K] int8: outputs whose mask byte is not positive are stored as zero
  uint32_t* sync;     // word 0: max |sum| of the launch (output), word 1: set when the wait gave up,
                      // words kSyncSlot0..: one slot per workgroup, max + 1; all zero on entry
  long long y8_bytes;
  int8_t* pool;       // optional [N,Q/2,Q/2,K] int8: 2x2 / stride-2 maximum of y8 (the max-pool that follows the layer)
  long long pool_bytes;
  // data gradient through a 2x2 / stride-2 max-pool in front of the layer: `mask` is the pooled map (this launch's
  // result is the gradient with respect to it), pool_x the pooling's input [N,2Q,2Q,K]; the rounded, masked result
  // goes to the position(s) of each window that equal the pooled value, into unpool [N,2Q,2Q,K], and y8 is not written
  const int8_t* pool_x;
  int8_t* unpool;
  long long unpool_bytes;
  int ties_all;
  int target_bits, method, trunc, bw_mode;
  const int32_t* rand;   // NITI_ROUND_STOCHASTIC: one random integer per output element [N,Q,Q,K], low `shift` bits used
  unsigned rq_flags;
  long long spin_limit;  // wall-clock ticks (100 MHz) the wait may last
  uint32_t* sticky;      // device-wide word set when the wait gives up, may be null
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
};
constexpr int kSyncSlot0 = 16;
// A grid with more workgroups than the device holds at once cannot wait for itself.  It runs as two launches of the
// same kernel instead (set by the launcher in rq_flags, not part of the interface):
//   kRqNoWait  every workgroup fills its slot (largest magnitude + 1, and next to it the shift it used), stores its
//              tile rounded with the predicted shift or what its own sums need, and ends;
//   kRqSettle  every workgroup first reads all slots - final after the first launch -, and ends at once if its tile
//              was stored with the final shift; otherwise it computes its tile again and stores it with that shift.
// With a good prediction (the previous training step's shift) the second launch does nothing but look.
constexpr unsigned kRqNoWait = 1u << 30, kRqSettle = 1u << 31;
static_assert(kSlotStride >= 2, "the two-launch form keeps the shift a tile was stored with in the word behind its slot");
constexpr int kMaxSlots = 4096;

// Q: image width = height; BR: output rows of one image per workgroup; NI: images per workgroup; BR*NI*Q == 256.
// The halo tile is NI*(BR+2) rows of Q slots of 32 bytes; for Q a multiple of 8 the bank of a slot depends on its
// column only, and the 16-byte halves of a slot are swapped where ((column >> 3) ^ row) is odd: 16 lanes reading
// consecutive columns of one row, or 8 + 8 columns of two adjacent rows, then hit 16 distinct bank groups.  The
// 4 x 4 maps of a deep network use the same code (16 whole images per workgroup) with some bank conflicts in
// their short rows; 2 x 2 maps have a kernel of their own below.
template <int Q, int BR, int NI, int KT>
struct HGeom {
  static constexpr int RP = Q;                             // no halo columns: horizontal neighbours come from lane shifts
  static_assert(Q == 4 || Q % 8 == 0, "rows of 4 or a multiple of 8 pixels");
  static constexpr int HR = BR + 2;
  static constexpr int SLOTS = NI * HR * RP;
  static constexpr int ACT_INSTR = (SLOTS + 31) / 32;      // one instruction fills 32 slots
  static constexpr int ACT_BYTES = ACT_INSTR * 1024;
  static constexpr int ACT_LOADS = (ACT_INSTR + 7) / 8;    // per wavefront per slice
  static constexpr int PX = BR * NI * Q;                   // output pixels per workgroup
  // 512 pixels x 64 channels: both halves of the workgroup's wavefronts work on the same 64 channels, each on 256 of
  // the pixels (for launches of the 64-channel tile with more workgroups than the device holds at once)
  static constexpr bool TWO = PX == 512;
  // KT == 32 (launches that would otherwise leave compute units idle): 8 wavefronts of 32 pixels x 32 channels
  static constexpr int PT = KT == 32 ? 1 : 2;              // 32-pixel tiles per wavefront
  static constexpr int NWF = TWO ? 2 : (KT == 32 ? 1 : KT / 64);   // 32-channel tiles per wavefront
  static constexpr int RPS = (KT <= 64 && !TWO) ? 3 : 1;   // filter rows per stage: the narrow tiles take a whole slice
  static constexpr int W_BYTES = RPS * 3 * KT * 32;        // one filter stage: RPS filter rows of three taps
  static constexpr int W_INSTR = W_BYTES / 1024;
  static constexpr int WSTAGES = 3;
  static constexpr int TILE_BYTES = 2 * ACT_BYTES + WSTAGES * W_BYTES;
  static constexpr int LDS_BYTES = TILE_BYTES + 1024;      // + dump slot / reduction words
  static_assert(PX == 256 || (PX == 512 && KT == 64), "a workgroup owns 256 output pixels, or 512 with the 64-channel tile");
  static_assert(KT == 32 || KT == 64 || KT == 128, "channel tile");
  static_assert(KT != 32 || Q <= 16, "the 32-channel tile's wavefronts own 32 pixels: whole 2 x 2 windows only up to 16-pixel rows");
  static_assert(NI == 1 || BR == Q, "several images per workgroup only as whole images");
};

// kWT: the filter operand is the FORWARD copy of the filter of the convolution whose data gradient this launch
// computes (input channels of this launch = that filter's output channels and vice versa, taps flipped); its
// 32 x 32 byte blocks are staged as they are and transposed by ds_read_b64_tr_b8 when the fragments are read.
// kSto: the requantising variant with StoShift (random integers read in the epilogue); instances of their own so that the
// others keep their register allocation.
template <int Q, int BR, int NI, int KT, bool kFused, bool kWT, bool kSto = false>
__global__ __launch_bounds__(512, 4) void conv3x3_halo_kernel(const HaloArgs a) {
  static_assert(kFused || !kSto);
  using G = HGeom<Q, BR, NI, KT>;
  constexpr int NWF = G::NWF;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t* const act_buf = smem;                         // 2 x ACT_BYTES
  int8_t* const w_buf = smem + 2 * G::ACT_BYTES;        // WSTAGES x W_BYTES
  int8_t* const dump = smem + G::TILE_BYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pixbase = blockIdx.x * G::PX;  // first output pixel of this workgroup in [N*Q*Q]
  const int kt = blockIdx.y;
  const int n0 = pixbase / (Q * Q);
  const int p0 = (pixbase - n0 * (Q * Q)) / Q;

  int settle_shift = -1;   // kRqSettle: the final shift, when this workgroup has to store its tile again
  if constexpr (kFused) {
    if ((a.rq_flags & kRqSettle) != 0) {
      uint32_t* const slots = a.sync + kSyncSlot0;
      uint32_t* const words = reinterpret_cast<uint32_t*>(dump);
      const int nb = gridDim.x * gridDim.y;
      const int b = blockIdx.y * gridDim.x + blockIdx.x;
      uint32_t m = 0;
      for (int i = tid; i < nb; i += 512) m = max(m, __hip_atomic_load(slot_word(slots, i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      m = wave_max_u32(m);
      if (lane == 0) words[wave] = m;
      __syncthreads();
      uint32_t g = words[0];
#pragma unroll
      for (int w = 1; w < 8; ++w) g = max(g, words[w]);
      const uint32_t gmax = g != 0u ? g - 1u : 0u;
      const int fshift = max(bitwidth_of(gmax, a.bw_mode) - a.target_bits, 0);
      const int used = static_cast<int>(slot_word(slots, b)[1]);
      if (b == 0 && tid == 0) {
        a.sync[0] = gmax;
        if (a.shift_out != nullptr) *a.shift_out = fshift;
        if (a.exp_out != nullptr) *a.exp_out = fshift + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
      }
      if (used == fshift) return;
      settle_shift = fshift;
      __syncthreads();   // the words are written again below
    }
  }

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.wp), 0, a.wp_bytes, 0x00020000);

  // NITI_RQ_SHIFT_HINT: *shift_out holds the caller's prediction (the previous training step's shift of this tensor).
  // Read here, a whole main loop before it is needed; workgroup (0, 0) overwrites the word only after all slots are
  // filled, i.e. after every workgroup has passed this line.
  // The load is unconditional (from the range word when there is no prediction), its address looks lane-dependent to
  // the compiler and its result is not looked at before the epilogue: a load inside a branch, or one whose result the
  // compiler knows to be the same in all lanes (and moves to a scalar register at once), would be waited for on the
  // spot - a trip to memory in front of the first stage's loads.
  bool hinted = false;
  int predicted_raw = 0;
  if constexpr (kFused) {
    hinted = (a.rq_flags & NITI_RQ_SHIFT_HINT) != 0 && a.shift_out != nullptr && settle_shift < 0;
    const int32_t* const src = hinted ? a.shift_out : reinterpret_cast<const int32_t*>(a.sync);
    predicted_raw = __hip_atomic_load(src + opaque_zero(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- activation staging: an instruction fills 32 consecutive slots; lane -> (slot lane/2, half lane%2).
  // A lane's offset is split into a part fixed for the whole launch (vector register) and the slice's 32 * cs
  // (scalar offset of the load), so a stage spends no vector arithmetic on it.  A lane with nothing to fetch
  // holds kOobFar, which no scalar offset below 2^31 brings back into range: the load then writes zeros.
  int act_off[G::ACT_LOADS];        // byte offset of this lane's 16 bytes for channel slice 0, or kOobFar
  int act_off_last[G::ACT_LOADS];   // the same for the last slice, whose upper 16 channels may not exist
  unsigned act_dst[G::ACT_LOADS];   // LDS byte address inside activation buffer 0, or the dump slot
  const unsigned act_lds = lds_addr(act_buf), w_lds = lds_addr(w_buf), dump_lds = lds_addr(dump);
#pragma unroll
  for (int i = 0; i < G::ACT_LOADS; ++i) {
    const int slot = (wave + 8 * i) * 32 + (lane >> 1);
    const int row = slot / G::RP, col = slot - row * G::RP;
    const int ni = row / G::HR, h = row - ni * G::HR;
    const int half = (lane & 1) ^ (((col >> 3) ^ row) & 1);
    const int ih = p0 + h - 1, iw = col;
    int off = kOobFar;
    if (slot < G::SLOTS && n0 + ni < a.N && ih >= 0 && ih < Q && iw >= 0 && iw < Q)
      off = (((n0 + ni) * Q + ih) * Q + iw) * a.C + half * 16;
    act_off[i] = off;
    act_off_last[i] = (a.cslices - 1) * 32 + half * 16 < a.C ? off : kOobFar;
    act_dst[i] = wave + 8 * i < G::ACT_INSTR ? act_lds + (wave + 8 * i) * 1024 : dump_lds;
  }
  auto issue_act = [&](int cs, int buf) {
    const bool last = cs == a.cslices - 1;
    const unsigned shift = buf * G::ACT_BYTES;
#pragma unroll
    for (int i = 0; i < G::ACT_LOADS; ++i) {
      const unsigned dst = wave + 8 * i < G::ACT_INSTR ? act_dst[i] + shift : act_dst[i];
      // through a local: with the array element written in the call itself the host pass of the compiler emitted no
      // launch stub for any instantiation of this kernel (the library then fails to load with an undefined symbol)
      const int off = last ? act_off_last[i] : act_off[i];
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, NITI_LDS_AT(dst), 16, off, cs * 32, 0, 0);
    }
  };
  // ---- filter staging.  The copy is [64-channel group][slice][tap][64 rows][32 bytes]: the three taps of a
  // filter row of one group are 6 KB in a row, the nine taps of a slice 18 KB.  A stage is W_INSTR load
  // instructions of 1 KB (KT == 128: one filter row of two groups, 12; KT == 64: a whole slice, 18); wavefront w
  // issues numbers w, w + 8, w + 16 as far as they exist.  The number of loads therefore differs between
  // wavefronts but never inside one (a lane-dependent condition around a load would let the compiler split it
  // into two instructions and break the vmcnt bookkeeping below).
  // A group beyond the last one (K not a multiple of 128) re-reads the last group instead of reading out of
  // range: its sums are never stored.
  const int ngroups = (a.K + 63) / 64;
  constexpr int WL = (G::W_INSTR + 7) / 8;               // filter loads per stage of the wavefronts that issue most
  const bool wfull = wave + 8 * (WL - 1) < G::W_INSTR;   // this wavefront is one of them; the others issue WL - 1
  static_assert(WL + G::ACT_LOADS <= 15);
  // kWT with one filter row per stage: a later row is an earlier tap, i.e. a step back of up to 6 taps; the lane's
  // part gives up those 6 taps (its smallest tap is 6) so that the scalar part never goes below zero
  constexpr int wback = (kWT && G::RPS == 1) ? 6 * 2048 : 0;
  auto w_src = [&](int q) {  // instruction q of a stage -> byte offset in the copy for slice 0, filter row 0
    if (kWT) {
      // KB q of a stage holds tap q / (KT/32) of the stage and 32-channel slice q % (KT/32) of this tile's output
      // channels: rows = 32 reduction channels (half a 64-row group of the forward copy), 32 bytes = 32 outputs
      const int cs = min(kt * (KT / 32) + q % (KT / 32), a.src_cslices - 1);
      return (cs * 9 + 8 - q / (KT / 32)) * 2048 + lane * 16 - wback;
    }
    if (KT == 32)   // instruction q = tap q: the tile's half (32 rows) of the 64-row group
      return min(kt >> 1, ngroups - 1) * a.cslices * (9 * 2048) + q * 2048 + (kt & 1) * 1024 + lane * 16;
    const int g = min(KT == 128 ? kt * 2 + q / 6 : kt, ngroups - 1);
    return g * a.cslices * (9 * 2048) + (KT == 128 ? q % 6 : q) * 1024 + lane * 16;
  };
  // The per-lane part of the three offsets is fixed for the launch; slice and filter row go into the scalar offset.
  const int wsrc_a = w_src(wave), wsrc_b = w_src(wave + 8), wsrc_c = w_src(wave + 16);
  const unsigned wdst = w_lds + wave * 1024;
  auto issue_w = [&](int cs, int r, int st) {
    // kWT: reduction slice cs = rows (cs & 1) * 32.. of group cs >> 1; a later filter row is an earlier forward tap
    const int rel =
        kWT ? (cs >> 1) * a.src_cslices * (9 * 2048) + (cs & 1) * 1024 - r * 3 * 2048 + wback : (cs * 9 + r * 3) * 2048;
    const unsigned dst = wdst + st * G::W_BYTES;
    if (wave < G::W_INSTR) __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS_AT(dst), 16, wsrc_a, rel, 0, 0);
    if (wave + 8 < G::W_INSTR)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS_AT(dst + 8 * 1024), 16, wsrc_b, rel, 0, 0);
    if (wave + 16 < G::W_INSTR)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS_AT(dst + 16 * 1024), 16, wsrc_c, rel, 0, 0);
  };

  // The first loads leave before the fragment addresses below are worked out (about half a microsecond of integer
  // arithmetic that the trip to memory can hide).  Per-wavefront load order, both pipelines: act(0), W(0), W(1).
  issue_act(0, 0);
  issue_w(0, 0, 0);
  if constexpr (G::RPS == 1) issue_w(0, 1, 1);
  else if (a.cslices > 1) issue_w(1, 0, 1);
  __builtin_amdgcn_sched_barrier(0);

  // ---- fragment addressing
  constexpr int PT = G::PT;
  const int wp_ = KT == 32 ? wave : (wave & 3);   // group of 32 PT pixels
  const int wc = KT == 32 ? 0 : (wave >> 2);      // channel group of KT/2 (TWO: pixel half, all wavefronts share the 64 channels)
  const int lr = lane & 31, lk = lane >> 5;
  constexpr int TAPB = (kWT || KT == 32) ? (KT / 32) * 1024 : 2048;   // bytes between consecutive taps inside a stage
  int w_addr[NWF][kWT ? 2 : 1];   // this lane's filter row(s) inside a stage, tap 0
#pragma unroll
  for (int i = 0; i < NWF; ++i) {
    if (kWT) {
      // block (tap, slice j) = [32 reduction rows][32 output bytes]; two transposing reads of 8 rows x 16 outputs
      const int j16 = lane & 15, gg = (lane >> 4) & 1;
      const int jslice = G::TWO ? i : (KT == 128 ? wc * 2 + i : wc);
#pragma unroll
      for (int o = 0; o < (kWT ? 2 : 1); ++o) {
        const int krow = 16 * lk + 8 * o + (j16 >> 1);
        w_addr[i][o] = jslice * 1024 + krow * 32 + ((gg ^ ((krow >> 3) & 1)) << 4) + 8 * (j16 & 1);
      }
    } else {
      // row inside the 64-channel group the stage holds at (KT == 128 ? wc * 6144 : 0)
      const int grow = (KT == 128 || G::TWO) ? i * 32 + lr : wc * 32 + lr;
      w_addr[i][0] = (KT == 128 ? wc * 6144 : 0) + grow * 32 + ((lk ^ ((grow >> 3) & 1)) << 4);
    }
  }
  int p_addr[PT];             // [pixel tile]: halo slot of this lane's pixel, filter row 0
#pragma unroll
  for (int j = 0; j < PT; ++j) {
    const int pix = (G::TWO ? wc * 256 : 0) + wp_ * (32 * PT) + j * 32 + lr;   // output pixel inside the workgroup's share
    const int prow = pix / Q, pw = pix % Q;        // row inside the workgroup's rows, column
    const int hrow = (prow / BR) * G::HR + (prow % BR);
    p_addr[j] = (hrow * G::RP + pw) * 32 + ((lk ^ (((pw >> 3) ^ hrow) & 1)) << 4);
  }
  // lanes whose left / right neighbour lies outside the image take the zero padding instead of the shifted value
  const int keep_l = (lr % Q) != 0 ? -1 : 0;
  const int keep_r = (lr % Q) != Q - 1 ? -1 : 0;

  v16i acc[NWF][PT];  // [channel tile][pixel tile]
#pragma unroll
  for (int i = 0; i < NWF; ++i)
#pragma unroll
    for (int j = 0; j < PT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  // one filter row: 12 (6) MFMAs from the activation tile sa and the three taps at sw
  auto filter_row = [&](const int8_t* sa, const int8_t* sw, int r, auto&& behind_first_tap) {
    const int roff = r * G::RP * 32;
    // pixels under the centre column of this filter row; the fragment layout is lane -> (pixel lane % 32,
    // 16 channels lane / 32), so the pixel to the left is one lane down and the one to the right one lane up
    v4i pc[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int at = (p_addr[j] + roff) ^ ((r & 1) << 4);
      if constexpr (kWT) pc[j] = lds_read_b128(lds_addr(sa) + at);   // counted by hand like the filter reads behind it
      else pc[j] = *reinterpret_cast<const v4i*>(sa + at);
    }
    v4i wf[3][NWF];
    v2i tlo[3][NWF], thi[3][NWF];   // kWT: halves of the transposed fragments until they have landed
    // order: centre tap (needs no shifting) first, then right, then left; wf[0] = tap s=1, wf[1] = s=2, wf[2] = s=0
    if constexpr (kWT) {
      const unsigned swa = lds_addr(sw);
      static_for<3>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        constexpr int off = ((s + 1) % 3) * TAPB;
#pragma unroll
        for (int i = 0; i < NWF; ++i) {
          tlo[s][i] = lds_read_tr8<off>(swa + w_addr[i][0]);
          thi[s][i] = lds_read_tr8<off>(swa + w_addr[i][kWT ? 1 : 0]);
        }
      });
    } else {
#pragma unroll
      for (int s = 0; s < 3; ++s)
#pragma unroll
        for (int i = 0; i < NWF; ++i) wf[s][i] = *reinterpret_cast<const v4i*>(sw + ((s + 1) % 3) * TAPB + w_addr[i][0]);
    }
    // kWT: the reads of a tap are 2 * NWF operations; those of the taps behind it may still be in flight
    auto tap_ready = [&](auto sc) {
      if constexpr (kWT) {
        constexpr int s = decltype(sc)::value;
        // the products of the tap before stay ahead of this wait (nothing else orders them against it)
        if (s > 0) __builtin_amdgcn_sched_barrier(0);
        lds_settle<(2 - s) * 2 * NWF>();
        if (s == 0) {
#pragma unroll
          for (int j = 0; j < PT; ++j) asm volatile("" : "+v"(pc[j]));
        }
#pragma unroll
        for (int i = 0; i < NWF; ++i) wf[s][i] = lds_landed(tlo[s][i], thi[s][i]);
      }
    };
    tap_ready(std::integral_constant<int, 0>{});
#pragma unroll
    for (int i = 0; i < NWF; ++i)
#pragma unroll
      for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[0][i], pc[j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    behind_first_tap();
    __builtin_amdgcn_sched_barrier(0);
    v4i ps[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j)
      ps[j] = shifted_and4<true>(pc[j], keep_r);
    tap_ready(std::integral_constant<int, 1>{});
#pragma unroll
    for (int i = 0; i < NWF; ++i)
#pragma unroll
      for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[1][i], ps[j], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int j = 0; j < PT; ++j)
      ps[j] = shifted_and4<false>(pc[j], keep_l);
    tap_ready(std::integral_constant<int, 2>{});
#pragma unroll
    for (int i = 0; i < NWF; ++i)
#pragma unroll
      for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[2][i], ps[j], acc[i][j], 0, 0, 0);
  };

  // A whole slice (three filter rows) from one stage, for the pipeline with one slice per stage.  All fragment reads
  // are inline assembly and run one filter row ahead of the products: row r + 1 is requested, then the wait leaves
  // exactly those requests in flight, then row r multiplies - so only the first row of a stage waits for LDS.  (Left
  // to itself the compiler keeps the fragments in few registers and alternates read, wait, product.)
  auto stage_rows = [&](unsigned saa, unsigned swa, auto&& behind_first_row) {
    constexpr int PER_TAP = NWF * (kWT ? 2 : 1);
    constexpr int ROW_READS = PT + 3 * PER_TAP;
    static_assert(ROW_READS <= 15, "the wait counter holds 15");
    v4i pcb[2][PT];
    v4i wfb[2][3][NWF];
    v2i tlo[2][3][NWF], thi[2][3][NWF];
    auto request = [&](auto rc) {
      constexpr int r = decltype(rc)::value;
      constexpr int b = r & 1;
#pragma unroll
      for (int j = 0; j < PT; ++j) pcb[b][j] = lds_read_b128_at<r * G::RP * 32>(saa + (p_addr[j] ^ ((r & 1) << 4)));
      static_for<3>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        constexpr int off = ((s + 1) % 3 + 3 * r) * TAPB;
#pragma unroll
        for (int i = 0; i < NWF; ++i) {
          if constexpr (kWT) {
            tlo[b][s][i] = lds_read_tr8<off>(swa + w_addr[i][0]);
            thi[b][s][i] = lds_read_tr8<off>(swa + w_addr[i][kWT ? 1 : 0]);
          } else {
            wfb[b][s][i] = lds_read_b128_at<off>(swa + w_addr[i][0]);
          }
        }
      });
    };
    request(std::integral_constant<int, 0>{});
    static_for<3>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      constexpr int b = r & 1;
      if constexpr (r < 2) request(std::integral_constant<int, r + 1>{});
      lds_settle<(r < 2) ? ROW_READS : 0>();
      v4i pc[PT], wf[3][NWF];
#pragma unroll
      for (int j = 0; j < PT; ++j) {
        pc[j] = pcb[b][j];
        asm volatile("" : "+v"(pc[j]));
      }
#pragma unroll
      for (int s = 0; s < 3; ++s)
#pragma unroll
        for (int i = 0; i < NWF; ++i) {
          if constexpr (kWT) {
            wf[s][i] = lds_landed(tlo[b][s][i], thi[b][s][i]);
          } else {
            wf[s][i] = wfb[b][s][i];
            asm volatile("" : "+v"(wf[s][i]));
          }
        }
#pragma unroll
      for (int i = 0; i < NWF; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[0][i], pc[j], acc[i][j], 0, 0, 0);
      v4i ps[PT];
#pragma unroll
      for (int j = 0; j < PT; ++j)
        ps[j] = shifted_and4<true>(pc[j], keep_r);
#pragma unroll
      for (int i = 0; i < NWF; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[1][i], ps[j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < PT; ++j)
        ps[j] = shifted_and4<false>(pc[j], keep_l);
#pragma unroll
      for (int i = 0; i < NWF; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[2][i], ps[j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);   // the next row's requests and wait stay behind these products
      if constexpr (r == 0) {
        behind_first_row();
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };

  __builtin_amdgcn_s_setprio(3);   // the main loop's instructions go ahead of a co-resident workgroup's epilogue
  if constexpr (G::RPS == 1) {
    // ---- pipeline, one filter row per stage.  Stage t = 3 * slice + filter row.  Per-wavefront load order: act(0),
    // W(0), W(1); inside stage t after its barrier: W(t+2), then - in the first stage of a slice - act(next slice).
    // Stage t needs W(t) (issued in stage t-2) and, in the first stage of a slice, that slice's activations
    // (issued three stages earlier, so older than W(t)).  Younger than W(t) are W(t+1) and the activation loads
    // issued in stage t-2 or t-1.
    const int nst = a.cslices * 3;
    for (int ci = 0; ci < a.cslices; ++ci) {
      const int8_t* sa = act_buf + (ci & 1) * G::ACT_BYTES;
      const bool more = ci + 1 < a.cslices;
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        const int t = ci * 3 + r;
        // younger than W(t): W(t+1) if there is one, and from the second stage of a slice on the next slice's
        // activations (issued in the first stage of this slice, after W(t) went out)
        if (r == 0 || !more) {
          if (r < 2 || more)
            hc_wait_vmcnt_pair<WL>(wfull);
          else
            hc_wait_vmcnt<0>();
        } else {
          hc_wait_vmcnt_pair<WL + G::ACT_LOADS>(wfull);
        }
        hc_sync();
        // the next loads go out behind the first tap's products (see the other pipeline below)
        filter_row(sa, w_buf + (t % G::WSTAGES) * G::W_BYTES, r, [&] {
          if (t + 2 < nst) {
            const int c2 = r == 0 ? ci : ci + 1, r2 = r == 0 ? 2 : r - 1;
            issue_w(c2, r2, (t + 2) % G::WSTAGES);
          }
          if (r == 0 && more) issue_act(ci + 1, (ci + 1) & 1);
        });
      }
    }
  } else {
    // ---- pipeline, one slice per stage (a barrier every 18 MFMAs instead of every 6).  Per-wavefront load order:
    // act(0), W(0), W(1); inside stage ci after its barrier: act(ci+1), then W(ci+2).  Stage ci needs W(ci) and
    // act(ci); the only loads younger than both are those of W(ci+1).
    for (int ci = 0; ci < a.cslices; ++ci) {
      const int8_t* sa = act_buf + (ci & 1) * G::ACT_BYTES;
      if (ci + 1 < a.cslices)
        hc_wait_vmcnt_pair<WL>(wfull);
      else
        hc_wait_vmcnt<0>();
      hc_sync();
      // The next loads go out behind the first filter row's products, not right behind the barrier: a wavefront
      // issues in order, the memory pipeline takes a few hundred clocks to accept a stage's load instructions (32-byte
      // pieces: 32 requests each), and right behind the barrier all eight wavefronts would spend them at the same
      // time with nothing queued on the matrix units.
      const int8_t* sw = w_buf + (ci % G::WSTAGES) * G::W_BYTES;
      stage_rows(lds_addr(sa), lds_addr(sw), [&] {
        if (ci + 1 < a.cslices) issue_act(ci + 1, (ci + 1) & 1);
        if (ci + 2 < a.cslices) issue_w(ci + 2, 0, (ci + 2) % G::WSTAGES);
      });
    }
  }

  // ---- epilogue: acc[i][j][4g+e] = channel kt*KT + wc*(KT/2) + i*32 + 8g + 4*lk + e of pixel pixbase+wp_*64+j*32+lr
  __builtin_amdgcn_s_setprio(0);
  const bool roundtrip = (a.flags & NITI_EPI_F32_ROUNDTRIP) != 0;
  int vmax = 0, vmin = 0;
#pragma unroll
  for (int i = 0; i < NWF; ++i)
#pragma unroll
    for (int j = 0; j < PT; ++j)
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
  const int chbase = G::TWO ? kt * KT : kt * KT + wc * (KT / 2);
  const int pixwave = pixbase + (G::TWO ? wc * 256 : 0) + wp_ * (32 * PT);   // first pixel of this wavefront
  uint32_t* const red = reinterpret_cast<uint32_t*>(dump);  // behind the tiles, clear of the patches below
  if constexpr (!kFused) {
    hc_sync();  // all wavefronts are done with the tiles: reuse LDS as per-wavefront transposition patches
    constexpr int ROWB = 32 * 4 + 16;  // one 32-channel tile row of int32, padded
    int8_t* patch = smem + wave * (32 * ROWB);
    const int rrow = lane >> 3, rcol = lane & 7;  // 8 lanes x 16 bytes = one 32-channel row
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
#pragma unroll
    for (int j = 0; j < PT; ++j) {
      const int mrow = pixwave + j * 32 + rrow;
#pragma unroll
      for (int i = 0; i < NWF; ++i) {
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
        const int ch = chbase + i * 32 + rcol * 4;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const v4i v = *reinterpret_cast<const v4i*>(patch + (t * 8 + rrow) * ROWB + rcol * 16);
          const int m = mrow + t * 8;
          const int off = (m < total_pix && ch < a.K) ? (m * a.K + ch) * 4 : kOob;
          __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, 2);
        }
      }
    }
    // one atomic per workgroup at most: same-address atomics serialise in the memory system
    if (a.absmax != nullptr) {
      const uint32_t wmax = wave_max_u32(lmax);
      if (lane == 0) red[wave] = wmax;
      __syncthreads();
      if (wave == 0) fold_absmax(a.absmax, lane < 8 ? red[lane] : 0u);
    }
  } else {
    // ---- tensor-wide range: workgroup maximum -> own slot -> maximum over the slots of all workgroups.
    // Results are stored before the range is final: the slots filled so far (read before this workgroup's own
    // maximum is known, so the latency hides behind that reduction) and the own maximum give a shift that is the
    // final one unless another workgroup raises the bit width; the int8 stores of all workgroups then overlap the
    // wait for the last slots instead of following it in one burst.  When the final shift differs, the sums (still
    // in registers) are rounded and stored once more.
    const int nb = gridDim.x * gridDim.y;
    uint32_t* const slots = a.sync + kSyncSlot0;
    constexpr int kLook = 8;   // slots a lane reads with its loads in flight together
    const bool nowait = (a.rq_flags & kRqNoWait) != 0;
    const bool settled = settle_shift >= 0;
    // Without a prediction, a hint: the first 64 * kLook slots as they are now.  With one the look would only put a
    // trip to memory between the last product and the first store.
    uint32_t early[kLook];
#pragma unroll
    for (int u = 0; u < kLook; ++u) {
      const int i = u * 64 + lane;
      early[u] = (wave == 0 && i < nb && !nowait && !settled && !hinted) ? __hip_atomic_load(slot_word(slots, i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    }
    const uint32_t wmax = wave_max_u32(lmax);
    __syncthreads();  // the tiles are dead from here on
    if (lane == 0) red[wave] = wmax;
    __syncthreads();
    if (wave == 0 && !settled) {
      uint32_t bmax = lane < 8 ? red[lane] : 0u;
      bmax = wave_max_u32(bmax);
      const int b = blockIdx.y * gridDim.x + blockIdx.x;
      if (lane == 0) __hip_atomic_store(slot_word(slots, b), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      uint32_t g = bmax + 1u;
#pragma unroll
      for (int u = 0; u < kLook; ++u) g = early[u] > g ? early[u] : g;
      g = wave_max_u32(g);
      if (lane == 0) {
        red[8] = g - 1u;
        red[9] = nb == 1 ? 1u : 0u;
      }
    }
    __syncthreads();
    // a shift below 1 means "no shift" whatever its value; the prediction counts unless this workgroup's own sums or
    // the slots seen so far already need more (or the range is final already)
    int shift = max(bitwidth_of(red[8], a.bw_mode) - a.target_bits, 0);
    bool final_range = red[9] != 0u;
    if (!final_range && hinted) shift = max(shift, predicted_raw);
    if (settled) shift = settle_shift;
    if (nowait) {   // the shift this tile is stored with, for the settling launch
      if (tid == 0) slot_word(slots, blockIdx.y * gridDim.x + blockIdx.x)[1] = static_cast<uint32_t>(shift);
    }
    final_range = final_range || nowait || settled;
    const bool trunc = a.trunc != 0;
    const bool relu = (a.rq_flags & NITI_RQ_RELU) != 0;
    const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
    // StoShift: the caller's random integer of each output element decides its rounding step; a tile that is rounded
    // twice (final shift unlike the first) takes the low bits of the same integers for the other shift
    constexpr bool sto = kSto;
    const __amdgpu_buffer_rsrc_t rrand = __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(a.rand), 0, sto ? a.y8_bytes * 4 : 0, 0x00020000);
    constexpr int PROW = NWF * 32 + 16;  // the wavefront's channels of one pixel, padded
    int8_t* patch = smem + wave * (32 * PT * PROW);
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y8, 0, a.y8_bytes, 0x00020000);
    constexpr int LPP = NWF * 2;       // lanes (16-byte pieces) per pixel
    constexpr int PPI = 64 / LPP;      // pixels per store instruction
    const int prow = lane / LPP, piece = lane % LPP;
    const int ch = chbase + piece * 16;
    if (rt) {   // once, in place: the values are rounded up to twice below
#pragma unroll
      for (int i = 0; i < NWF; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = f32_roundtrip(acc[i][j][e]);
    }
    // The mask bytes (ReLU backward of the layer below / the pooled map) do not depend on the rounding: the first two
    // of the wavefront's pieces are requested here and each later one two pieces ahead of its use, so that they have
    // arrived when the stores below need them - requested where it is used, every piece would be a trip to memory
    // between two stores.
    // (Only where registers allow: the wavefronts with four accumulator tiles are at the 128-register limit of two
    // workgroups per CU and fetch each piece where it is used.)
    constexpr int NPIECE = 32 * PT / PPI;
    constexpr bool kMaskAhead = NWF * PT <= 2;
    constexpr int MKD = !kMaskAhead ? 1 : (NPIECE < 2 ? NPIECE : 2);
    v4i mkpre[MKD];
    auto mask_request = [&](int t) {
      const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.mask), 0, a.y8_bytes, 0x00020000);
      const int m = pixwave + t * PPI + prow;
      const int off = (m < total_pix && ch < a.K) ? m * a.K + ch : kOob;
      mkpre[t % MKD] = __builtin_amdgcn_raw_buffer_load_b128(rm, off, 0, 0);
    };
    // the same for the pooling windows of the folded max-pool backward, one piece ahead
    v4i xwpre[kMaskAhead ? 4 : 1];
    auto window_offsets = [&](int t, int (&wo)[4]) {
      const int m = pixwave + t * PPI + prow;
      const bool in = m < total_pix && ch < a.K;
      const int n = m / (Q * Q), rem = m - n * (Q * Q);
      const int pp = rem / Q, pq = rem - pp * Q;
      const int rowb = 2 * Q * a.K;
      const int base = ((n * 2 * Q + 2 * pp) * 2 * Q + 2 * pq) * a.K + ch;
#pragma unroll
      for (int k = 0; k < 4; ++k) wo[k] = in ? base + (k >> 1) * rowb + (k & 1) * a.K : kOob;
    };
    auto window_request = [&](int t) {
      if constexpr (kMaskAhead) {
        const __amdgpu_buffer_rsrc_t rxp = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.pool_x), 0, a.unpool_bytes, 0x00020000);
        int wo[4];
        window_offsets(t, wo);
#pragma unroll
        for (int k = 0; k < 4; ++k) xwpre[k] = __builtin_amdgcn_raw_buffer_load_b128(rxp, wo[k], 0, 0);
      }
    };
    if (kMaskAhead && a.mask != nullptr) {
#pragma unroll
      for (int t = 0; t < MKD; ++t) mask_request(t);
      if (a.unpool != nullptr) window_request(0);
    }
#pragma nounroll
    for (int pass = 0; pass < 2; ++pass) {
      // the sums look modified to the compiler in every pass: nothing derived from them (magnitudes, signs) is
      // computed ahead of the loop and kept in 64 more registers
#pragma unroll
      for (int i = 0; i < NWF; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j) asm volatile("" : "+v"(acc[i][j]));
      // round, pack four channels per dword, transpose through a per-wavefront patch, store 16-byte pieces; the
      // common rounding mode gets a short form
      // The shift is the same in every lane but has come through LDS, which the compiler cannot know: made a scalar
      // here, the choice between the two forms below is ONE scalar branch.  (Left inside the loops as a per-lane
      // condition it cost every value both forms' set-up under execution masks and a taken branch.)
      const int ushift = __builtin_amdgcn_readfirstlane(shift);
      const bool fast = ushift >= 1 && !trunc && !psto && !sto;
      const int sm1 = ushift - 1, lo = relu ? 0 : -127;
      auto round_tiles = [&](auto fastc) {
        constexpr bool kFast = decltype(fastc)::value;
#pragma unroll
        for (int j = 0; j < PT; ++j)
#pragma unroll
          for (int i = 0; i < NWF; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              uint32_t packed;
              if constexpr (kFast) {
                packed = round4_nearest_floor_fast(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3], sm1, lo);
              } else {
                int r[4];
                v4i u = {0, 0, 0, 0};
                if (sto) {   // the four values are consecutive channels of one pixel
                  const int m = pixwave + j * 32 + lr, c0 = chbase + i * 32 + 8 * g + 4 * lk;
                  u = __builtin_amdgcn_raw_buffer_load_b128(rrand, (m < total_pix && c0 < a.K) ? (m * a.K + c0) * 4 : kOob, 0, 0);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const int x = acc[i][j][4 * g + e];
                  if (ushift >= 1)
                    r[e] = sto    ? round_sto32(x, ushift, trunc, u[e])
                           : psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, ushift, trunc)
                                  : round_one32<NITI_ROUND_NEAREST>(x, ushift, trunc);
                  else r[e] = wrap_to_i8(x);
                  if (relu && r[e] < 0) r[e] = 0;
                }
                packed = pack4_i8(r[0], r[1], r[2], r[3]);
              }
              *reinterpret_cast<uint32_t*>(patch + (j * 32 + lr) * PROW + (i * 8 + 2 * g + lk) * 4) = packed;
            }
      };
      if (fast) round_tiles(std::true_type{});
      else round_tiles(std::false_type{});
      // same wavefront reads back what it wrote: LDS operations of one wavefront complete in order
#pragma unroll
      for (int t = 0; t < 32 * PT / PPI; ++t) {
        const int pl = t * PPI + prow;
        v4i v = *reinterpret_cast<const v4i*>(patch + pl * PROW + piece * 16);
        const int m = pixwave + pl;
        const int off = (m < total_pix && ch < a.K) ? m * a.K + ch : kOob;
        v4i mk;
        if (a.mask != nullptr) {  // ReLU backward of the layer below, folded in: its output is this layer's input
          if constexpr (kMaskAhead) {
            mk = mkpre[t % MKD];
            if (t + MKD < NPIECE) mask_request(t + MKD);
          } else {
            const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.mask), 0, a.y8_bytes, 0x00020000);
            mk = __builtin_amdgcn_raw_buffer_load_b128(rm, off, 0, 0);
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] &= static_cast<int>(positive_bytes(static_cast<uint32_t>(mk[q])));
        }
        if (a.unpool != nullptr) {
          // max-pool backward folded in (mk holds the pooled values): the window of pooled pixel m in the pooling's input
          const __amdgpu_buffer_rsrc_t rxp = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.pool_x), 0, a.unpool_bytes, 0x00020000);
          const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(a.unpool, 0, a.unpool_bytes, 0x00020000);
          int wo[4];
          window_offsets(t, wo);
          v4i xw[4], ow[4];
          if constexpr (kMaskAhead) {
#pragma unroll
            for (int k = 0; k < 4; ++k) xw[k] = xwpre[k];
            if (t + 1 < NPIECE) window_request(t + 1);
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) xw[k] = __builtin_amdgcn_raw_buffer_load_b128(rxp, wo[k], 0, 0);
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint32_t taken = 0;   // bytes whose gradient an earlier position of the window (scan order) already received
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const uint32_t eq = equal_bytes(static_cast<uint32_t>(xw[k][q]), static_cast<uint32_t>(mk[q]));
              const uint32_t keep = a.ties_all != 0 ? eq : eq & ~taken;
              ow[k][q] = static_cast<int>(static_cast<uint32_t>(v[q]) & keep);
              taken |= eq;
            }
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) __builtin_amdgcn_raw_buffer_store_b128(ow[k], ru, wo[k], 0, 0);
        } else {
          // the 128-channel tile writes 64 bytes per pixel and wavefront: streaming stores start the write-back of the
          // 16 MiB result while the kernel still runs (measured 2 us per launch); the 32-byte pieces of the 64-channel
          // tile are slower that way
          __builtin_amdgcn_raw_buffer_store_b128(v, ry, off, 0, NWF == 2 ? 2 : 0);
        }
      }
      if (a.pool != nullptr) {
        // The max-pool behind this layer, from the rounded values still in the patch: the wavefront's 64 pixels are a
        // strip of whole image rows (or whole images), i.e. 16 whole 2 x 2 windows; a lane takes 16 channels of one.
        constexpr int PC = Q / 2;   // pooled pixels per row
        const int pq = lane / LPP;
        if (pq < 8 * PT) {
          const int l0 = 2 * (pq / PC) * Q + 2 * (pq % PC);   // upper left pixel of the window inside the strip
          const int8_t* src = patch + l0 * PROW + piece * 16;
          const v4i p00 = *reinterpret_cast<const v4i*>(src), p01 = *reinterpret_cast<const v4i*>(src + PROW);
          const v4i p10 = *reinterpret_cast<const v4i*>(src + Q * PROW), p11 = *reinterpret_cast<const v4i*>(src + (Q + 1) * PROW);
          v4i mx;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            mx[q] = static_cast<int>(max_i8x4(max_i8x4(static_cast<uint32_t>(p00[q]), static_cast<uint32_t>(p01[q])),
                                              max_i8x4(static_cast<uint32_t>(p10[q]), static_cast<uint32_t>(p11[q]))));
          const int m0 = pixwave + l0;
          const int n = m0 / (Q * Q), rem = m0 - n * (Q * Q);
          const int pr = rem / Q, pcol = rem - pr * Q;
          const int pix2 = (n * PC + (pr >> 1)) * PC + (pcol >> 1);
          const int off = (m0 < total_pix && ch < a.K) ? pix2 * a.K + ch : kOob;
          const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(a.pool, 0, a.pool_bytes, 0x00020000);
          __builtin_amdgcn_raw_buffer_store_b128(mx, rp, off, 0, 0);
        }
      }
      if (final_range) break;
      // ---- wait for the slots of all workgroups; the maximum over them is the tensor's range
      if (wave == 0) {
        const uint32_t g = wait_slots(slots, nb, a.spin_limit, &a.sync[1], a.sticky);
        if (lane == 0) red[8] = g != 0u ? g - 1u : 0u;
      }
      __syncthreads();
      final_range = true;
      const int fshift = max(bitwidth_of(red[8], a.bw_mode) - a.target_bits, 0);
      if (fshift == shift) break;
      shift = fshift;
      __builtin_amdgcn_s_waitcnt(0);   // the stores of the first pass leave before those that replace them
      if (kMaskAhead && a.mask != nullptr) {
#pragma unroll
        for (int t = 0; t < MKD; ++t) mask_request(t);
        if (a.unpool != nullptr) window_request(0);
      }
    }
    if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0 && !nowait && !settled) {
      const int sh = shift > 0 ? shift : 0;
      a.sync[0] = red[8];
      if (a.shift_out != nullptr) *a.shift_out = sh;
      if (a.exp_out != nullptr)
        *a.exp_out = sh + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
    }
  }
}

// ---- 2 x 2 maps -----------------------------------------------------------------------------------------
// With one pixel of padding every output pixel of a 2 x 2 map sees all four input pixels, each through one filter
// tap: the convolution is a dense product [N] x [4 C] x [4 K] whose filter operand for output pixel p and input
// pixel q is tap (qy - py + 1, qx - px + 1).  The halo kernel would give such a layer (the last ones of a deep
// network: few pixels, many channels) one workgroup per 64 images and spend 5 of its 9 taps on padding; here a
// workgroup owns 32 images x 32 output channels, wavefront (p, half) computes output pixel p over one half of the
// channel slices, and the two halves are added through LDS.  Both operands are fetched as MFMA fragments without a
// shared tile: the activation rows straight into registers, the filter from the same prepared copy the halo kernel
// reads (a 32 x 32 block of it is 1 KB in a row) - into registers, or, for the data gradient reading the forward
// copy, into a per-wavefront LDS slot that ds_read_b64_tr_b8 transposes.  Loads run eight reduction steps ahead.
constexpr int kMap2Depth = 8;                               // reduction steps with their loads in flight, per wavefront
constexpr int kMap2RedBytes = 4 * 64 * 16 * 4;              // sums of the second reduction half
constexpr int kMap2StageBytes = 8 * kMap2Depth * 1024;      // kWT: filter blocks in flight, all wavefronts
constexpr int kMap2ActMaxC = 512;                           // kLdsAct: input channels whose activations fit in LDS
constexpr size_t map2_fixed_lds(bool wt) { return static_cast<size_t>(kMap2RedBytes) + 64 + (wt ? kMap2StageBytes : 0); }
// kLdsAct: the workgroup's activations (32 images x 4 pixels x C) behind the rest, rows of 4 C + 16 bytes (the 16
// spread the 32 images of a fragment read over the banks)
constexpr size_t map2_lds_bytes(bool wt, int act_c) { return map2_fixed_lds(wt) + (act_c > 0 ? static_cast<size_t>(32) * (4 * act_c + 16) : 0); }

// kLdsAct: the four wavefronts of a reduction half multiply the same activation fragments (with different taps), so
// the workgroup stages its activations in LDS once and every wavefront reads its fragments there: 1.25 KB instead of
// 2 KB per step come through the vector memory path, which is what bounds this kernel.
template <bool kFused, bool kWT, bool kLdsAct>
__global__ __launch_bounds__(512) void conv3x3_map2_kernel(const HaloArgs a, int itiles) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int* const red = reinterpret_cast<int*>(smem);                                      // [p][4][64] x 16 bytes
  uint32_t* const words = reinterpret_cast<uint32_t*>(smem + kMap2RedBytes);          // 4 maxima, the range
  int8_t* const act_s = smem + map2_fixed_lds(kWT);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p = wave & 3, rh = wave >> 2;
  const int lr = lane & 31, lk = lane >> 5;
  // consecutive workgroups go to consecutive dies: give each die a contiguous range of tiles, so that the tiles
  // sharing a block of the filter (same output channels) read it through one L2
  const int nb = gridDim.x;
  const int b = (nb & 7) == 0 ? (blockIdx.x & 7) * (nb >> 3) + (blockIdx.x >> 3) : blockIdx.x;
  const int kt = b / itiles, it = b - kt * itiles;      // 32-channel tile, 32-image tile
  const int n = it * 32 + lr;

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.wp), 0, a.wp_bytes, 0x00020000);

  // this wavefront's channel slices and its reduction steps (slice, input pixel)
  const int half0 = (a.cslices + 1) >> 1;
  const int cs0 = rh == 0 ? 0 : half0;
  const int nsteps = (rh == 0 ? half0 : a.cslices - half0) * 4;
  const int py = p >> 1, px = p & 1;
  const int a_base = n < a.N ? n * 4 * a.C + lk * 16 : kOob;
  // filter fragment of this lane inside a 1 KB block (32 rows of 32 bytes, 16-byte halves swapped in odd groups of 8 rows)
  int w_frag[2];
  if (kWT) {
    const int j16 = lane & 15, gg = (lane >> 4) & 1;
#pragma unroll
    for (int o = 0; o < 2; ++o) {
      const int krow = 16 * lk + 8 * o + (j16 >> 1);
      w_frag[o] = krow * 32 + ((gg ^ ((krow >> 3) & 1)) << 4) + 8 * (j16 & 1);
    }
  } else {
    w_frag[0] = w_frag[1] = lr * 32 + ((lk ^ ((lr >> 3) & 1)) << 4);
  }
  int8_t* const stage = smem + kMap2RedBytes + 64 + wave * (kMap2Depth * 1024);

  const int act_pitch = 4 * a.C + 16;
  if (kLdsAct) {
    // rows = images, 4 C bytes each (the four pixels in a row); 16-byte pieces, coalesced
    const int pieces = a.C >> 2;                          // 16-byte pieces of an image: 4 pixels x C / 16
    for (int i = tid; i < 32 * pieces; i += 512) {
      const int img = i / pieces, pc = i - img * pieces;
      const int nn = it * 32 + img;
      const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rx, nn < a.N ? nn * 4 * a.C + pc * 16 : kOob, 0, 0);
      *reinterpret_cast<v4i*>(act_s + img * act_pitch + pc * 16) = v;
    }
    __syncthreads();
  }
  const int8_t* const act_lane = act_s + lr * act_pitch + lk * 16;
  v4i fa[kMap2Depth], fw[kMap2Depth];
  // Loads of step s into slot u.  Steps past the wavefront's last one are issued all the same, with out-of-range
  // offsets (zeros, no memory traffic): the loop body is free of branches, so the number of loads in flight behind
  // any load is a constant - for the compiler's wait counts as for those written by hand below.
  auto issue = [&](int s, int u) {
    const int cs = cs0 + (s >> 2), q = s & 3;
    const int tap = ((q >> 1) - py + 1) * 3 + (q & 1) - px + 1;
    const bool live = s < nsteps;
    int aoff = kOob;
    if (live && a_base != kOob && cs * 32 + lk * 16 < a.C) aoff = a_base + q * a.C + cs * 32;
    if (!kLdsAct) fa[u] = __builtin_amdgcn_raw_buffer_load_b128(rx, aoff, 0, 0);
    if (kWT) {
      // forward copy [reduction group of 64][this launch's output slice][flipped tap][64 rows][32 bytes]
      const int blk = (((cs >> 1) * a.src_cslices + kt) * 9 + 8 - tap) * 2048 + (cs & 1) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rw, NITI_LDS(stage + u * 1024), 16, live ? blk + lane * 16 : kOob, 0, 0, 0);
      asm volatile("" ::: "memory");   // both loads leave here, in this order
    } else {
      const int blk = (((kt >> 1) * a.cslices + cs) * 9 + tap) * 2048 + (kt & 1) * 1024;
      fw[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, live ? blk + w_frag[0] : kOob, 0, 0);
    }
  };

  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
#pragma unroll
  for (int u = 0; u < kMap2Depth; ++u) issue(u, u);
  for (int base = 0; base < nsteps; base += kMap2Depth) {
#pragma unroll
    for (int u = 0; u < kMap2Depth; ++u) {
      if (kWT) {
        // two loads per step (one with the activations in LDS), completing in order: all but those of the seven younger
        // steps have landed
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((kLdsAct ? 1 : 2) * (kMap2Depth - 1)));
        asm volatile("" ::: "memory");
        const unsigned src = lds_addr(stage + u * 1024);
        const v2i lo = lds_read_tr8<0>(src + w_frag[0]);
        const v2i hi = lds_read_tr8<0>(src + w_frag[1]);
        lds_settle<0>();   // also: the slot is read out before the next block is sent to it
        fw[u] = lds_landed(lo, hi);
      }
      if (kLdsAct) {
        const int st = base + u;                             // steps past the last one read slice 0 (their filter fragments are zero)
        const int cs = st < nsteps ? cs0 + (st >> 2) : 0;
        fa[u] = *reinterpret_cast<const v4i*>(act_lane + (st & 3) * a.C + cs * 32);
      }
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[u], fa[u], acc, 0, 0, 0);
      issue(base + u + kMap2Depth, u);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // the (empty) loads issued ahead of the last steps
  asm volatile("" ::: "memory");

  // ---- add the two reduction halves: acc[4g + e] = channel kt*32 + 8g + 4*lk + e of image n, pixel p
  if (rh == 1) {
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<v4i*>(red + ((p * 4 + g) * 64 + lane) * 4) = v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
  }
  __syncthreads();
  const bool roundtrip = (a.flags & NITI_EPI_F32_ROUNDTRIP) != 0;
  if (rh == 0) {
    uint32_t lmax = 0;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const v4i o = *reinterpret_cast<const v4i*>(red + ((p * 4 + g) * 64 + lane) * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int v = acc[4 * g + e] + o[e];
        if (roundtrip) v = f32_roundtrip(v);
        acc[4 * g + e] = v;
        const uint32_t m = uabs(v);
        lmax = m > lmax ? m : lmax;
      }
    }
    lmax = wave_max_u32(lmax);
    if (lane == 0) words[wave] = lmax;
  }
  __syncthreads();
  const long long row = (static_cast<long long>(n) * 4 + p) * a.K;   // first output element of (image, pixel)
  const int ch = kt * 32 + 4 * lk;                                   // + 8g
  if constexpr (!kFused) {
    if (rh == 0) {
      const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int c = ch + 8 * g;
        const int off = (n < a.N && c < a.K) ? static_cast<int>((row + c) * 4) : kOob;
        __builtin_amdgcn_raw_buffer_store_b128(v4i{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]}, ry, off, 0, 0);
      }
    }
    if (a.absmax != nullptr && wave == 0) fold_absmax(a.absmax, lane < 4 ? words[lane] : 0u);
  } else {
    // ---- tensor-wide range: workgroup maximum -> own slot -> maximum over the slots of all workgroups
    if (wave == 0) {
      uint32_t bmax = lane < 4 ? words[lane] : 0u;
      bmax = wave_max_u32(bmax);
      uint32_t* const slots = a.sync + kSyncSlot0;
      if (lane == 0) __hip_atomic_store(slot_word(slots, blockIdx.x), bmax + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t g = wait_slots(slots, nb, a.spin_limit, &a.sync[1], a.sticky);
      if (lane == 0) words[4] = g != 0u ? g - 1u : 0u;
    }
    __syncthreads();
    const uint32_t gmax = words[4];
    // a scalar, so that the choice of rounding form below is a scalar branch (see the kernel above)
    const int shift = __builtin_amdgcn_readfirstlane(max(bitwidth_of(gmax, a.bw_mode) - a.target_bits, 0));
    if (rh == 0) {
      const bool trunc = a.trunc != 0;
      const bool relu = (a.rq_flags & NITI_RQ_RELU) != 0;
      const bool psto = a.method == NITI_ROUND_PSEUDO_STOCHASTIC;
      const bool fast = shift >= 1 && !trunc && !psto;
      const int sm1 = shift - 1, lo = relu ? 0 : -127;
      const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y8, 0, a.y8_bytes, 0x00020000);
      const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.mask != nullptr ? a.mask : a.y8), 0, a.y8_bytes, 0x00020000);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t v;
        if (fast) {
          v = round4_nearest_floor_fast(acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3], sm1, lo);
        } else {
          int r[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int x = acc[4 * g + e];
            if (shift >= 1) r[e] = psto ? round_one32<NITI_ROUND_PSEUDO_STOCHASTIC>(x, shift, trunc) : round_one32<NITI_ROUND_NEAREST>(x, shift, trunc);
            else r[e] = wrap_to_i8(x);
            if (relu && r[e] < 0) r[e] = 0;
          }
          v = pack4_i8(r[0], r[1], r[2], r[3]);
        }
        const int c = ch + 8 * g;
        const int off = (n < a.N && c < a.K) ? static_cast<int>(row + c) : kOob;
        uint32_t mk = 0;
        if (a.mask != nullptr) {   // ReLU backward of the layer below, folded in: its output is this layer's input
          mk = static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b32(rm, off, 0, 0));
          v &= positive_bytes(mk);
        }
        if (a.unpool != nullptr) {
          // max-pool backward folded in (mk holds the pooled values): the window of this pixel in the pooling's 4 x 4 input
          const __amdgpu_buffer_rsrc_t rxp = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.pool_x), 0, a.unpool_bytes, 0x00020000);
          const __amdgpu_buffer_rsrc_t ru = __builtin_amdgcn_make_buffer_rsrc(a.unpool, 0, a.unpool_bytes, 0x00020000);
          const int base = ((n * 4 + 2 * py) * 4 + 2 * px) * a.K + c;
          int wo[4];
          uint32_t xw[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) wo[q] = off == kOob ? kOob : base + (q >> 1) * 4 * a.K + (q & 1) * a.K;
#pragma unroll
          for (int q = 0; q < 4; ++q) xw[q] = static_cast<uint32_t>(__builtin_amdgcn_raw_buffer_load_b32(rxp, wo[q], 0, 0));
          uint32_t taken = 0;   // bytes whose gradient an earlier position of the window (scan order) already received
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t eq = equal_bytes(xw[q], mk);
            const uint32_t keep = a.ties_all != 0 ? eq : eq & ~taken;
            taken |= eq;
            __builtin_amdgcn_raw_buffer_store_b32(v & keep, ru, wo[q], 0, 0);
          }
        } else {
          __builtin_amdgcn_raw_buffer_store_b32(v, ry, off, 0, 0);
        }
        if (a.pool != nullptr) reinterpret_cast<uint32_t*>(red)[(p * 4 + g) * 64 + lane] = v;   // the sums parked here have been read
      }
    }
    if (a.pool != nullptr) {
      // the 2 x 2 max-pool behind this layer leaves one pixel: wavefront g takes the maximum over the four pixels for
      // its group of channels
      __syncthreads();
      if (rh == 0) {
        const uint32_t* pv = reinterpret_cast<const uint32_t*>(red);
        const int g = p;
        const uint32_t mx = max_i8x4(max_i8x4(pv[(0 * 4 + g) * 64 + lane], pv[(1 * 4 + g) * 64 + lane]),
                                     max_i8x4(pv[(2 * 4 + g) * 64 + lane], pv[(3 * 4 + g) * 64 + lane]));
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(a.pool, 0, a.pool_bytes, 0x00020000);
        const int c = ch + 8 * g;
        __builtin_amdgcn_raw_buffer_store_b32(mx, rp, (n < a.N && c < a.K) ? n * a.K + c : kOob, 0, 0);
      }
    }
    if (blockIdx.x == 0 && tid == 0) {
      a.sync[0] = gmax;
      if (a.shift_out != nullptr) *a.shift_out = shift;
      if (a.exp_out != nullptr) *a.exp_out = shift + (a.exp_a != nullptr ? *a.exp_a : 0) + (a.exp_b != nullptr ? *a.exp_b : 0);
    }
  }
}

// Filter arrangement for the kernel above.  mode 0 (forward): F(k, tap, c) = w[k][tap][c], w is [K][9][C].
// mode 1 (data gradient): the roles of the channel dimensions swap and the taps flip:
// F(k', tap, c') = w[c'][8 - tap][k'], with k' < C and c' < K of the original filter.
// dst[kg][cs][tap][row][half ^ ((row >> 3) & 1)][16] = F(kg*64 + row, tap, cs*32 + half*16 ..), zero outside.
__global__ __launch_bounds__(256) void halo_filter_prepare_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ dst,
                                                                  int kout, int cin, int mode, int64_t total) {
  const int cslices = (cin + 31) / 32;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int b = static_cast<int>(i & 15);
    const int ppos = static_cast<int>((i >> 4) & 1);
    const int row = static_cast<int>((i >> 5) & 63);
    int64_t t = i >> 11;
    const int tap = static_cast<int>(t % 9);
    t /= 9;
    const int cs = static_cast<int>(t % cslices);
    const int kg = static_cast<int>(t / cslices);
    const int half = ppos ^ ((row >> 3) & 1);
    const int k = kg * 64 + row;
    const int c = cs * 32 + half * 16 + b;
    int8_t v = 0;
    if (k < kout && c < cin) {
      if (mode == 0) v = w[(static_cast<int64_t>(k) * 9 + tap) * cin + c];
      else v = w[(static_cast<int64_t>(c) * 9 + (8 - tap)) * kout + k];
    }
    dst[i] = v;
  }
}

// Channel tile of a launch: 128 unless that leaves fewer workgroups than the device runs at once while
// a tile of 64 would give it more to do.
int halo_ktile(long long pix, int K, int H, int C) {
  static int cus_of[kDeviceSlots] = {};
  int& cus = cus_of[device_slot()];
  if (cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
  }
  const char* e = getenv("NITI_HALO_KT");  // tests and tuning runs pin the tile
  const int forced = e != nullptr ? atoi(e) : 0;
  if (forced == 128 || forced == 64) return forced;
  if (forced == 32 && H <= 16) return 32;
  // fewer 64-channel tiles than compute units on the small maps: tiles of 32 channels, twice as many workgroups
  if (forced == 0 && H <= 8 && K > 32 && (pix / 256) * ((K + 63) / 64) < cus) return 32;
  // exactly one 64-channel tile per compute unit and a short reduction: two 32-channel workgroups per unit overlap
  // each other's fill and epilogue (measured per launch: 128 -> 256 at 16 x 16 data gradient 14.5 -> 13.9 us, 256 -> 512
  // at 8 x 8 forward 13.9 -> 12.7 us; with 512 input channels the narrower tile's longer loop loses more than that)
  if (forced == 0 && H <= 16 && K > 32 && C <= 256 && (pix / 256) * ((K + 63) / 64) == cus) return 32;
  if (K <= 64) return 64;   // nothing to gain from computing 128 channels
  // one slice of reduction (the first layer): the launch is all output stores, and the 64-channel tile's workgroups -
  // 512 pixels each where 256-pixel ones would not all fit - spread them better (3 -> 128 at 32 x 32: 9.9 -> 9.5 us)
  if (forced == 0 && C <= 32 && H == 32 && pix % 512 == 0) return 64;
  const long long b128 = (pix / 256) * ((K + 127) / 128);
  return (b128 < 2LL * cus && K > 64) ? 64 : 128;
}

// The 64-channel tile with 512 pixels per workgroup: where 256-pixel workgroups would be more than the device holds
// at once (a condition of the requantising variant), on the large maps where such launches occur.
bool halo_two_pixel_tiles(long long pix, int K, int H, int ktile) {
  if (ktile != 64 || (H != 32 && H != 16) || pix % 512 != 0) return false;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  return (pix / 256) * ((K + 63) / 64) > 2LL * cus;
}

template <int Q, int BR, int NI, int KT, bool kFused, bool kWT, bool kSto = false>
int launch_halo(const HaloArgs& a, hipStream_t stream) {
  using G = HGeom<Q, BR, NI, KT>;
  constexpr size_t lds = G::LDS_BYTES;
  static_assert(8 * 32 * (32 * 4 + 16) <= G::TILE_BYTES, "int32 patches must stay clear of the reduction words");
  static_assert(8 * 32 * G::PT * (G::NWF * 32 + 16) <= G::TILE_BYTES, "int8 patches must stay clear of the reduction words");
  static_assert(2 * lds <= 160 * 1024, "two workgroups per compute unit");
  auto k = conv3x3_halo_kernel<Q, BR, NI, KT, kFused, kWT, kSto>;
  static bool attr_set_of[kDeviceSlots] = {};   // function attributes are per device
  static int resident_of[kDeviceSlots] = {};     // workgroups the device holds at once
  const int slot = device_slot();
  bool& attr_set = attr_set_of[slot];
  int& resident = resident_of[slot];
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
  dim3 grid(static_cast<unsigned>((pix + G::PX - 1) / G::PX), (a.K + KT - 1) / KT);
  if (kFused && static_cast<long long>(grid.x) * grid.y > resident) {
    // more workgroups than the device holds at once: nobody waits; a second launch settles the tiles stored with
    // another shift than the final one
    if (static_cast<long long>(grid.x) * grid.y > kMaxSlots)
      return fail(NITI_ERR_UNSUPPORTED, "conv3x3_halo: %u workgroups exceed the %d range slots", grid.x * grid.y, kMaxSlots);
    HaloArgs b = a;
    b.rq_flags = a.rq_flags | kRqNoWait;
    hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, b);
    b.rq_flags = a.rq_flags | kRqSettle;
    hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, b);
    return check_launch("conv3x3_halo");
  }
  hipLaunchKernelGGL(k, grid, dim3(512), lds, stream, a);
  return check_launch("conv3x3_halo");
}

inline int map2_blocks(int N, int K) { return ((N + 31) / 32) * ((K + 31) / 32); }

template <bool kFused, bool kWT, bool kLdsAct>
int launch_map2_as(const HaloArgs& a, hipStream_t stream) {
  constexpr size_t lds = map2_lds_bytes(kWT, kLdsAct ? kMap2ActMaxC : 0);
  auto k = conv3x3_map2_kernel<kFused, kWT, kLdsAct>;
  static bool attr_set_of[kDeviceSlots] = {};   // function attributes are per device
  static int resident_of[kDeviceSlots] = {};     // workgroups the device holds at once
  const int slot = device_slot();
  bool& attr_set = attr_set_of[slot];
  int& resident = resident_of[slot];
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "conv3x3_map2: cannot reserve %zu bytes of LDS", lds);
    if (kFused) {
      int dev = 0, cus = 0, per_cu = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
          hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(k), 512, lds) != hipSuccess)
        return fail(NITI_ERR_LAUNCH, "conv3x3_map2: cannot query occupancy");
      resident = cus * per_cu;
    }
    attr_set = true;
  }
  const int itiles = (a.N + 31) / 32;
  const int nb = map2_blocks(a.N, a.K);
  if (kFused && nb > resident) {
    // the variant with its activations in LDS holds fewer workgroups per compute unit: the direct loads may still fit
    if constexpr (kLdsAct) return launch_map2_as<kFused, kWT, false>(a, stream);
    return fail(NITI_ERR_UNSUPPORTED, "conv3x3_map2: %d workgroups do not fit on the device at once (%d)", nb, resident);
  }
  hipLaunchKernelGGL(k, dim3(nb), dim3(512), lds, stream, a, itiles);
  return check_launch("conv3x3_map2");
}

template <bool kFused, bool kWT>
int launch_map2(const HaloArgs& a, hipStream_t stream) {
  // activations through LDS where a workgroup's share fits (NITI_MAP2_LDS=0 pins the direct loads)
  const char* e = getenv("NITI_MAP2_LDS");
  if (a.C <= kMap2ActMaxC && a.C % 32 == 0 && (e == nullptr || e[0] != '0')) return launch_map2_as<kFused, kWT, true>(a, stream);
  return launch_map2_as<kFused, kWT, false>(a, stream);
}

template <bool kFused, bool kWT, bool kSto = false>
int launch_halo_tiles(const HaloArgs& a, int H, hipStream_t stream) {
  if (H == 2) return launch_map2<kFused, kWT>(a, stream);
  const int ktile = halo_ktile(static_cast<long long>(a.N) * H * H, a.K, H, a.C);
  if (ktile == 128) {
    if (H == 32) return launch_halo<32, 8, 1, 128, kFused, kWT, kSto>(a, stream);
    if (H == 16) return launch_halo<16, 16, 1, 128, kFused, kWT, kSto>(a, stream);
    if (H == 8) return launch_halo<8, 8, 4, 128, kFused, kWT, kSto>(a, stream);
    return launch_halo<4, 4, 16, 128, kFused, kWT, kSto>(a, stream);
  }
  if (ktile == 32) {
    if (H == 16) return launch_halo<16, 16, 1, 32, kFused, kWT, kSto>(a, stream);
    if (H == 8) return launch_halo<8, 8, 4, 32, kFused, kWT, kSto>(a, stream);
    return launch_halo<4, 4, 16, 32, kFused, kWT, kSto>(a, stream);
  }
  if constexpr (kFused) {
    if (halo_two_pixel_tiles(static_cast<long long>(a.N) * H * H, a.K, H, ktile)) {
      if (H == 32) return launch_halo<32, 16, 1, 64, kFused, kWT, kSto>(a, stream);
      return launch_halo<16, 16, 2, 64, kFused, kWT, kSto>(a, stream);
    }
  }
  if (H == 32) return launch_halo<32, 8, 1, 64, kFused, kWT, kSto>(a, stream);
  if (H == 16) return launch_halo<16, 16, 1, 64, kFused, kWT, kSto>(a, stream);
  if (H == 8) return launch_halo<8, 8, 4, 64, kFused, kWT, kSto>(a, stream);
  return launch_halo<4, 4, 16, 64, kFused, kWT, kSto>(a, stream);
}

template <bool kFused>
int launch_halo_any(const HaloArgs& a, int H, hipStream_t stream) {
  if constexpr (kFused) {
    if (a.method == NITI_ROUND_STOCHASTIC)
      return a.src_cslices > 0 ? launch_halo_tiles<true, true, true>(a, H, stream) : launch_halo_tiles<true, false, true>(a, H, stream);
  }
  return a.src_cslices > 0 ? launch_halo_tiles<kFused, true>(a, H, stream) : launch_halo_tiles<kFused, false>(a, H, stream);
}

void fill_common(HaloArgs& a, const int8_t* x, const int8_t* wp, int N, int H, int C, int K, unsigned flags) {
  // NITI_CONV_FILTER_FORWARD_COPY: wp is the forward copy of the [C][3][3][K] filter whose data gradient this is
  a = HaloArgs{};
  a.x = x;
  a.wp = wp;
  a.N = N;
  a.C = C;
  a.K = K;
  a.cslices = (C + 31) / 32;
  a.x_bytes = static_cast<long long>(N) * H * H * C;
  const bool wt = (flags & NITI_CONV_FILTER_FORWARD_COPY) != 0;
  a.src_cslices = wt ? (K + 31) / 32 : 0;
  a.wp_bytes = static_cast<long long>(wt ? conv3x3_halo_filter_bytes(K, C) : conv3x3_halo_filter_bytes(C, K));
  a.flags = flags;
}

}  // namespace

bool conv3x3_halo_supported(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (R != 3 || S != 3 || stride != 1 || pad != 1 || H != W) return false;
  if (H != 2 && H != 4 && H != 8 && H != 16 && H != 32) return false;
  if (C % 16 != 0 || K % 4 != 0) return false;
  const long long pix = static_cast<long long>(N) * H * W;
  if (H != 2 && pix % 256 != 0) return false;  // workgroups own whole rows / whole images (2 x 2 maps: any batch)
  if (pix * C >= 0x7fffffffLL || pix * K * 4 >= 0x7fffffffLL) return false;
  if (conv3x3_halo_filter_bytes(C, K) >= 0x7fffffffULL) return false;
  return true;
}

size_t conv3x3_halo_filter_bytes(int C, int K) {
  return static_cast<size_t>((K + 63) / 64) * ((C + 31) / 32) * 9 * 64 * 32;
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
  fill_common(a, x, wp, N, H, C, K, flags);
  a.y = y;
  a.absmax = absmax;
  a.y_bytes = static_cast<long long>(N) * H * H * K * 4;
  return launch_halo_any<false>(a, H, stream);
}

// Workgroups of a launch of the requantising variant (= sync slots), or 0 when the variant cannot run the shape.
int conv3x3_halo_requant_blocks(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (!conv3x3_halo_supported(N, H, W, C, K, R, S, stride, pad) || K % 16 != 0) return 0;
  const long long pix = static_cast<long long>(N) * H * W;
  const int ktile = halo_ktile(pix, K, H, C);
  const long long px = halo_two_pixel_tiles(pix, K, H, ktile) ? 512 : 256;
  const long long nb = H == 2 ? map2_blocks(N, K) : (pix / px) * ((K + ktile - 1) / ktile);
  return nb <= kMaxSlots ? static_cast<int>(nb) : 0;  // more than the device holds at once run as two launches
}

size_t conv3x3_halo_sync_words(int blocks) { return static_cast<size_t>(kSyncSlot0) + slot_words(blocks); }

int launch_conv3x3_halo_requant(const int8_t* x, const int8_t* wp, int8_t* y8, int N, int H, int C, int K, unsigned flags,
                                uint32_t* sync, const RequantSpec& rq, hipStream_t stream) {
  HaloArgs a;
  fill_common(a, x, wp, N, H, C, K, flags);
  a.y8 = y8;
  a.mask = rq.mask;
  a.sync = sync;
  a.y8_bytes = static_cast<long long>(N) * H * H * K;
  a.pool = rq.pool;
  a.pool_bytes = static_cast<long long>(N) * (H / 2) * (H / 2) * K;
  a.pool_x = rq.pool_x;
  a.unpool = rq.unpool;
  a.unpool_bytes = 4 * a.y8_bytes;
  a.ties_all = rq.ties_all;
  if (a.unpool != nullptr) {
    if (a.mask == nullptr || a.pool_x == nullptr) return fail(NITI_ERR_INVALID_ARG, "conv_requant: unpooling needs the pooled map and the pooling's input");
    if (a.unpool_bytes >= 0x7fffffffLL) return fail(NITI_ERR_UNSUPPORTED, "conv_requant: unpooled map of 2 GiB or more");
  }
  a.target_bits = rq.target_bits;
  a.method = rq.method;
  a.trunc = rq.trunc;
  a.bw_mode = rq.bw_mode;
  a.rand = rq.rand;
  if (rq.method == NITI_ROUND_STOCHASTIC) {
    if (rq.rand == nullptr) return fail(NITI_ERR_INVALID_ARG, "conv_requant: stochastic rounding needs the random integers");
    if (H == 2 || a.unpool != nullptr)
      return fail(NITI_ERR_UNSUPPORTED, "conv_requant: stochastic rounding is not folded in on 2 x 2 maps or with the pooling's backward pass; use the two-pass path");
  }
  a.rq_flags = rq.flags;
  a.spin_limit = rq.spin_limit;
  a.sticky = rq.sticky;
  a.shift_out = rq.shift_out;
  a.exp_a = rq.exp_a;
  a.exp_b = rq.exp_b;
  a.exp_out = rq.exp_out;
  return launch_halo_any<true>(a, H, stream);
}

}  // namespace niti
