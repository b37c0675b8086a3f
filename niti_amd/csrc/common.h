// Shared declarations of the gfx950 library: status plumbing, vector types, small device helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "niti_gfx950.h"

#ifndef NITI_SLOT_STRIDE
#define NITI_SLOT_STRIDE 4
#endif
// bytes of the kernel-ready filter copy that niti_conv2d_i8_fprop_requant_static can hold in the library's own array
#ifndef NITI_STATIC_FILTER_BYTES
#define NITI_STATIC_FILTER_BYTES (4u << 20)
#endif

namespace niti {

// Launch set-up that holds per device (a kernel's function attributes, how many workgroups the device holds at
// once) is cached in arrays of this many entries, indexed by device_slot().
constexpr int kDeviceSlots = 64;
inline int device_slot() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
  return dev % kDeviceSlots;
}


typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Records a message for niti_last_error() and returns `status`.
int fail(int status, const char* fmt, ...);
void clear_error();

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NITI_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return NITI_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__device__ inline bool aligned16_dev(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ceil(log2(r)) as integer arithmetic (0 for r <= 1)
__host__ __device__ inline int bitwidth_exact(uint32_t r) {
  if (r <= 1) return 0;
  uint32_t v = r - 1;
#if defined(__HIP_DEVICE_COMPILE__)
  return 32 - __clz(v);
#else
  return 32 - __builtin_clz(v);
#endif
}

// int(ceil(log2f((float)r))) under a correctly rounded log2f.  (float)r = 2^e * (1 + j*2^-23);
// the sum e + log2(1 + j*2^-23) rounds back to e exactly when j is at most jmax(e): half an ulp
// of e, expressed in mantissa steps (0, 0, 1, 2, 5 for e in [1,2), [2,4), [4,8), [8,16), [16,32)).
__host__ __device__ inline int bitwidth_float32(uint32_t r) {
  if (r == 0) return 0;
  float f = static_cast<float>(r);  // round to nearest even
  union { float f; uint32_t u; } cvt;
  cvt.f = f;
  const int e = static_cast<int>((cvt.u >> 23) & 0xFF) - 127;
  const uint32_t j = cvt.u & 0x7FFFFFu;
  if (j == 0) return e;
  if (e <= 0) return e + 1;
  int t = 0;
  for (int v = e; v > 1; v >>= 1) ++t;
  const uint32_t jmax = t >= 4 ? 5u : (t == 3 ? 2u : (t == 2 ? 1u : 0u));
  return j <= jmax ? e : e + 1;
}

__host__ __device__ inline int bitwidth_of(uint32_t r, int bw_mode) {
  return bw_mode == NITI_BW_F32 ? bitwidth_float32(r) : bitwidth_exact(r);
}

// int32 -> fp32 (round to nearest even) -> int32 with saturation: the reference's CUTLASS
// LinearCombinationClamp<int32, 4, int32, float> epilogue with alpha = 1, beta = 0.
__device__ inline int f32_roundtrip(int v) {
  const float f = static_cast<float>(v);
  if (f >= 2147483648.0f) return 2147483647;
  return static_cast<int>(f);  // f is integral and >= -2^31 here
}

// Zero that the compiler cannot see through: added to a uniform address it keeps a load's result in a vector
// register (a result known to be uniform is moved to a scalar register right behind the load, which waits for it).
__device__ inline int opaque_zero() {
  int z;
  asm volatile("v_mov_b32 %0, 0" : "=v"(z));
  return z;
}

__device__ inline uint32_t uabs(int v) { return v < 0 ? 0u - static_cast<uint32_t>(v) : static_cast<uint32_t>(v); }

// Largest value over the wavefront, in every lane.  A max-scan inside each row of 16 lanes (row_shr 1, 2, 4, 8: lanes
// without a source keep the neutral 0), then the row totals carried into the following rows (row_bcast 15 and 31),
// which leaves the wavefront's maximum in lane 63: six data-parallel moves instead of six trips through the LDS
// crossbar.
__device__ inline uint32_t wave_max_u32(uint32_t v) {
  uint32_t o;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x111, 0xf, 0xf, false));
  v = o > v ? o : v;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x112, 0xf, 0xf, false));
  v = o > v ? o : v;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x114, 0xf, 0xf, false));
  v = o > v ? o : v;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x118, 0xf, 0xf, false));
  v = o > v ? o : v;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x142, 0xa, 0xf, false));
  v = o > v ? o : v;
  o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x143, 0xc, 0xf, false));
  v = o > v ? o : v;
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}

// Range exchange between the resident workgroups of a launch: workgroup b stores (its maximum + 1) in slot b and
// reads all slots.  Slots are kSlotStride words apart: the 4-byte stores of all workgroups arrive within a
// microsecond and are serialised per memory channel, so the slots are spread over more of them.
constexpr int kSlotStride = NITI_SLOT_STRIDE;
__device__ inline uint32_t* slot_word(uint32_t* slots, int b) { return slots + static_cast<long long>(b) * kSlotStride; }
inline size_t slot_words(int blocks) { return static_cast<size_t>((blocks + 15) / 16 * 16) * kSlotStride; }

// Called by a whole wavefront: waits until all nb slots are filled and returns the largest value.  512 slots at a
// time, eight per lane with the loads in flight together (one trip to memory per look); a lane reads a slot again
// only while it is still empty, so the reads of the waiting workgroups die down as the slots fill.  Gives up after
// spin_limit ticks of the 100 MHz clock: `code` is or-ed into *timed_out (the launch's own flag: 1 = a wait for the
// tensor-wide range, 2 = the one-launch weight gradient's wait for the partial sums), *sticky (the device-wide word
// that niti_sync_timeouts reads, may be null) is set to 1 and the largest value seen so far is returned.  A limit of
// zero gives up after the first look whatever it saw (tests of this path: every waiting wavefront then takes it).
__device__ inline uint32_t wait_slots(uint32_t* slots, int nb, long long spin_limit, uint32_t* timed_out, uint32_t* sticky,
                                      uint32_t code = 1u) {
  constexpr int kLook = 8;
  const int lane = threadIdx.x & 63;
  const long long t0 = wall_clock64();
  uint32_t g = 0;
  bool gave_up = false;
  for (int base = 0; base < nb && !gave_up; base += 64 * kLook) {
    uint32_t v[kLook];
#pragma unroll
    for (int u = 0; u < kLook; ++u) v[u] = base + u * 64 + lane < nb ? 0u : 1u;
    for (;;) {
      uint32_t t[kLook];
#pragma unroll
      for (int u = 0; u < kLook; ++u)
        t[u] = v[u] == 0u ? __hip_atomic_load(slot_word(slots, base + u * 64 + lane), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : v[u];
      bool ok = true;
#pragma unroll
      for (int u = 0; u < kLook; ++u) {
        v[u] = t[u];
        ok = ok && v[u] != 0u;
      }
      if (__all(ok) && spin_limit > 0) break;
      if (spin_limit <= 0 || wall_clock64() - t0 > spin_limit) {
        if (lane == 0) {
          __hip_atomic_fetch_or(timed_out, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (sticky != nullptr) __hip_atomic_store(sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        gave_up = true;
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
#pragma unroll
    for (int u = 0; u < kLook; ++u) g = v[u] > g ? v[u] : g;
  }
  return wave_max_u32(g);
}

// Folds a wavefront's max |value| into *dst.  Same-address atomics serialise in the memory
// system (about 10 ns each), so a wavefront first looks at the value already there and only
// issues the atomic when it would raise it; the stored value only ever grows, so a stale read
// can at worst cause a redundant atomic.
__device__ inline void fold_absmax(uint32_t* dst, uint32_t lane_max) {
  const uint32_t m = wave_max_u32(lane_max);
  if ((threadIdx.x & 63) == 0 && m != 0) {
    const uint32_t seen = __hip_atomic_load(dst, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (m > seen) atomicMax(dst, m);
  }
}

// ---- launchers implemented in the .hip files ----
struct ConvProblem {
  const int8_t* x;   // [N,H,W,C]
  const int8_t* w;   // [K,R,S,C]
  int32_t* y;        // element (n,p,q,k) lives at n*ysN + p*ysP + q*ysQ + k*ysK
  uint32_t* absmax;  // may be null
  int N, H, W, C, K, R, S, stride, pad;
  long long ysN, ysP, ysQ, ysK;
  int split_k;       // 1: plain stores; >1: k-range split, int32 atomic adds into zeroed y
  unsigned flags;
};
int launch_conv_igemm(const ConvProblem& p, hipStream_t stream);

// int32 GEMM of operands with a slow reduction index (NN: b as [k][n]; TN: a as [k][m] too; TT: a as [k][m], b as
// [n][k]), read as stored
bool gemm_kmajor_shape(int trans_a, int trans_b, int m, int n, int k);
size_t gemm_kmajor_workspace(int trans_a, int trans_b, int m, int n, int k);   // partial sums of a reduction split over workgroups
int launch_gemm_kmajor(int trans_a, int trans_b, const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k, bool roundtrip,
                       uint32_t* absmax, void* workspace, hipStream_t stream);

int launch_fill_u32(uint32_t* dst, int64_t n, uint32_t value, hipStream_t stream);
// dst[c][r][s][k] = w[k][R-1-r][S-1-s][c]
int launch_filter_flip_transpose(const int8_t* w, int8_t* dst, int K, int R, int S, int C, hipStream_t stream);
// src [A][B][C] int8 -> dst [C][B][Apad], zero filled for a >= A
int launch_transpose_outer_inner_i8(const int8_t* src, int8_t* dst, int A, int B, int C, int Apad, hipStream_t stream);
// in place: v = roundtrip(v) if requested; absmax folded if non-null
int launch_post_i32(int32_t* v, int64_t n, bool roundtrip, uint32_t* absmax, hipStream_t stream);

// native 3x3 / stride 1 / pad 1 weight gradient (wgrad3x3.hip)
bool wgrad3x3_supported(int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
size_t wgrad3x3_workspace(int N, int H, int C, int K);
int launch_wgrad3x3(const int8_t* act, const int8_t* err, int32_t* dw, int N, int H, int C, int K, bool roundtrip,
                    uint32_t* absmax, void* workspace, hipStream_t stream);

// 3x3 / stride 1 / pad 1 forward kernel with LDS-resident activation halo (conv3x3_halo.hip)
bool conv3x3_halo_supported(int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
size_t conv3x3_halo_filter_bytes(int C, int K);
int launch_halo_filter_prepare(const int8_t* w, int8_t* dst, int kout, int cin, int mode, hipStream_t stream);
int launch_conv3x3_halo(const int8_t* x, const int8_t* wp, int32_t* y, int N, int H, int C, int K, unsigned flags,
                        uint32_t* absmax, hipStream_t stream);
// requantisation parameters of the convolution that rounds its own sums to int8
struct RequantSpec {
  int target_bits, method, trunc, bw_mode;
  unsigned flags;          // NITI_RQ_*
  long long spin_limit;    // 100 MHz wall-clock ticks the grid-wide wait may last
  uint32_t* sticky;        // device-wide word set when a wait gives up (timeout_word()), may be null
  int32_t* shift_out;
  const int32_t* exp_a;
  const int32_t* exp_b;
  int32_t* exp_out;
  const int8_t* mask;      // conv + requantisation only: optional ReLU-backward mask, laid out like the output
  int8_t* pool;            // forward conv + requantisation only: optional 2x2 / stride-2 maximum of the output
  // data gradient only: fold in the backward pass of a 2x2 / stride-2 max-pool in front of the layer (mask = pooled map)
  const int8_t* pool_x = nullptr;   // the pooling's input [N,2H,2W,C]
  int8_t* unpool = nullptr;         // result [N,2H,2W,C] (the [N,H,W,C] output is then not written)
  int ties_all = 0;
  const int32_t* rand = nullptr;    // conv + requantisation with NITI_ROUND_STOCHASTIC: one integer per output element
};
// wall-clock ticks (100 MHz) a grid-wide wait may last (api.hip)
long long sync_spin_limit();
// this device's word that every grid-wide wait sets when it gives up (api.hip); nullptr if it cannot be looked up
uint32_t* timeout_word();
int wgrad3x3_finish_blocks(int C, int K);
size_t wgrad3x3_sync_words(int blocks);
int launch_wgrad3x3_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int H, int C, int K,
                           bool roundtrip, uint32_t* sync, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep,
                           void* workspace, hipStream_t stream);
// one-launch weight gradient + update of the first layer (wgrad_first.hip); its accumulation buffer are extra zeroed sync
// words behind the finishing kernel's
size_t wgrad_first_extra_words(int H, int C, int K);
bool wgrad_first_supported(int N, int H, int C, int K, int w_channels);
int launch_wgrad_first_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int K, bool roundtrip,
                              uint32_t* sync, int32_t* accum, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep,
                              hipStream_t stream);
// one-launch weight gradient + update for 4 x 4 and 2 x 2 maps (wgrad_small.hip); sync words as for the finishing kernel
bool wgrad_small_shape(int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
bool wgrad_small_supported(int N, int H, int C, int K, int w_channels);
int launch_wgrad_small_update(const int8_t* act, const int8_t* err, int8_t* w, int N, int H, int C, int K, bool roundtrip,
                              uint32_t* sync, const RequantSpec& rq, int8_t* g8, int32_t* dw, int8_t* wprep, hipStream_t stream);
int conv3x3_halo_requant_blocks(int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
size_t conv3x3_halo_sync_words(int blocks);
int launch_conv3x3_halo_requant(const int8_t* x, const int8_t* wp, int8_t* y8, int N, int H, int C, int K, unsigned flags,
                                uint32_t* sync, const RequantSpec& rq, hipStream_t stream);

}  // namespace niti
