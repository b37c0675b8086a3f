// extern "C" surface of libniti_gfx950: argument checking, workspace carving and the
// composition of kernels behind each entry point declared in include/niti_gfx950.h.
#include <stdarg.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "common.h"

namespace niti {
namespace {
thread_local char g_err[512] = {0};

__global__ void pad_rows_i8_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst, int64_t rows, int k, int kpad) {
  const int64_t total = rows * kpad;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / kpad;
    const int c = static_cast<int>(i - r * kpad);
    dst[i] = c < k ? src[r * k + c] : static_cast<int8_t>(0);
  }
}

inline size_t round256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
inline int round16(int v) { return (v + 15) & ~15; }

int pick_split(long long tiles, int kiters) {
  // aim at ~3 workgroups per compute unit, keep at least 8 main-loop steps per slice
  long long want = (768 + tiles - 1) / tiles;
  long long maxs = kiters / 8;
  if (maxs < 1) maxs = 1;
  if (want > maxs) want = maxs;
  if (want < 1) want = 1;
  return static_cast<int>(want);
}
}  // namespace

int fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return status;
}
void clear_error() { g_err[0] = 0; }

}  // namespace niti

using namespace niti;

extern "C" int niti_version(void) { return 100; }

extern "C" const char* niti_status_string(int status) {
  switch (status) {
    case NITI_OK: return "ok";
    case NITI_ERR_INVALID_ARG: return "invalid argument";
    case NITI_ERR_UNSUPPORTED: return "unsupported shape";
    case NITI_ERR_WORKSPACE: return "workspace too small";
    case NITI_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

extern "C" const char* niti_last_error(void) { return g_err; }

extern "C" int niti_bitwidth(uint32_t r, int bw_mode) { return bitwidth_of(r, bw_mode); }

extern "C" int niti_fill_u32(uint32_t* dst, int64_t n, uint32_t value, void* stream) {
  clear_error();
  if (n < 0 || (n > 0 && dst == nullptr)) return fail(NITI_ERR_INVALID_ARG, "fill: bad arguments");
  return launch_fill_u32(dst, n, value, static_cast<hipStream_t>(stream));
}

static int check_conv_dims(const char* who, int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0)
    return fail(NITI_ERR_INVALID_ARG, "%s: non-positive extent (N=%d H=%d W=%d C=%d K=%d R=%d S=%d)", who, N, H, W, C, K, R, S);
  if (stride <= 0 || pad < 0) return fail(NITI_ERR_INVALID_ARG, "%s: stride=%d pad=%d", who, stride, pad);
  if (H + 2 * pad < R || W + 2 * pad < S) return fail(NITI_ERR_INVALID_ARG, "%s: filter larger than padded input", who);
  return NITI_OK;
}

// bits outside `allowed` are refused rather than ignored: a caller built against a newer header finds out at once
static int check_flags(const char* who, unsigned flags, unsigned allowed) {
  if ((flags & ~allowed) != 0u) return fail(NITI_ERR_INVALID_ARG, "%s: flags=%#x (accepted: %#x)", who, flags, allowed);
  return NITI_OK;
}

static bool halo_off() {
  static const bool off = [] {   // read once (initialisation of a function-local static is thread-safe)
    const char* e = getenv("NITI_NO_HALO");
    return e != nullptr && e[0] == '1';
  }();
  return off;
}

// which filter copy a convolution of this shape uses: 0 none (w as stored), 1 flipped/transposed
// [C][R][S][K] (data gradient through the generic kernel), 2 / 3 tap-major blocks of the halo kernel
// (forward / data gradient)
static int filter_copy_kind(int N, int H, int W, int C, int K, int R, int S, int stride, int pad, int dgrad) {
  if (!dgrad) return (!halo_off() && conv3x3_halo_supported(N, H, W, C, K, R, S, stride, pad)) ? 2 : 0;
  if (stride != 1 || R != S || pad > R - 1) return 1;
  const int P = H + 2 * pad - R + 1, Q = W + 2 * pad - S + 1;
  return (!halo_off() && conv3x3_halo_supported(N, P, Q, K, C, R, S, 1, R - 1 - pad)) ? 3 : 1;
}

// NITI_CONV_FILTER_FORWARD_COPY is for a data gradient whose forward pass and whose own launch both run the halo
// kernel (the copy of kind 2 is then read in place of the copy of kind 3); anything else is a caller error
static int check_forward_copy_flag(const char* who, int dgrad, unsigned flags, int N, int H, int W, int C, int K, int R, int S,
                                   int stride, int pad) {
  if (!(flags & NITI_CONV_FILTER_FORWARD_COPY)) return NITI_OK;
  if (!dgrad) return fail(NITI_ERR_INVALID_ARG, "%s: NITI_CONV_FILTER_FORWARD_COPY is a data-gradient flag", who);
  if (!(flags & NITI_CONV_FILTER_PREPARED))
    return fail(NITI_ERR_INVALID_ARG, "%s: NITI_CONV_FILTER_FORWARD_COPY needs NITI_CONV_FILTER_PREPARED", who);
  if (filter_copy_kind(N, H, W, C, K, R, S, stride, pad, 0) != 2 || filter_copy_kind(N, H, W, C, K, R, S, stride, pad, 1) != 3)
    return fail(NITI_ERR_UNSUPPORTED, "%s: the forward filter copy serves the data gradient only where both run the 3x3 kernel", who);
  return NITI_OK;
}

extern "C" int niti_pad_rows_i8(const int8_t* src, int8_t* dst, int64_t rows, int k, int kpad, void* stream) {
  clear_error();
  if (src == nullptr || dst == nullptr) return fail(NITI_ERR_INVALID_ARG, "pad_rows: null pointer");
  if (rows <= 0 || k <= 0 || kpad < k) return fail(NITI_ERR_INVALID_ARG, "pad_rows: rows=%lld k=%d kpad=%d", static_cast<long long>(rows), k, kpad);
  int64_t g = (rows * kpad + 255) / 256;
  if (g > 4096) g = 4096;
  hipLaunchKernelGGL(pad_rows_i8_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0, static_cast<hipStream_t>(stream), src, dst, rows, k, kpad);
  return check_launch("pad_rows");
}

extern "C" size_t niti_conv2d_i8_filter_workspace(int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                                                  int dgrad) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || stride <= 0 || pad < 0) return 0;
  switch (filter_copy_kind(N, H, W, C, K, R, S, stride, pad, dgrad)) {
    case 1: return round256(static_cast<size_t>(C) * R * S * K);
    case 2: return conv3x3_halo_filter_bytes(C, K);
    case 3: return conv3x3_halo_filter_bytes(K, C);
    default: return 0;
  }
}

extern "C" int niti_conv2d_i8_filter_prepare(const int8_t* w, int8_t* dst, size_t dst_bytes, int N, int H, int W, int C,
                                             int K, int R, int S, int stride, int pad, int dgrad, void* stream) {
  clear_error();
  int st = check_conv_dims("filter_prepare", N, H, W, C, K, R, S, stride, pad);
  if (st != NITI_OK) return st;
  const size_t need = niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, pad, dgrad);
  if (need == 0) return NITI_OK;
  if (w == nullptr || dst == nullptr || dst_bytes < need || !aligned16(dst))
    return fail(NITI_ERR_WORKSPACE, "filter_prepare: needs %zu bytes (16-byte aligned), got %zu", need, dst_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (filter_copy_kind(N, H, W, C, K, R, S, stride, pad, dgrad)) {
    case 1: return launch_filter_flip_transpose(w, dst, K, R, S, C, s);
    case 2: return launch_halo_filter_prepare(w, dst, K, C, 0, s);
    case 3: return launch_halo_filter_prepare(w, dst, C, K, 1, s);
    default: return NITI_OK;
  }
}

extern "C" int niti_conv2d_i8_fprop(const int8_t* x, const int8_t* w, int32_t* y, int N, int H, int W, int C, int K,
                                    int R, int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  clear_error();
  int st = check_conv_dims("conv_fprop", N, H, W, C, K, R, S, stride, pad);
  if (st == NITI_OK) st = check_flags("conv_fprop", flags, NITI_EPI_F32_ROUNDTRIP | NITI_CONV_FILTER_PREPARED);
  if (st != NITI_OK) return st;
  if (x == nullptr || w == nullptr || y == nullptr) return fail(NITI_ERR_INVALID_ARG, "conv_fprop: null pointer");
  if (!aligned16(x) || !aligned16(w) || !aligned16(y)) return fail(NITI_ERR_INVALID_ARG, "conv_fprop: pointers must be 16-byte aligned");
  if (C % 16 != 0) return fail(NITI_ERR_UNSUPPORTED, "conv: C=%d must be a multiple of 16", C);
  st = check_forward_copy_flag("conv_fprop", 0, flags, N, H, W, C, K, R, S, stride, pad);
  if (st != NITI_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int kind = filter_copy_kind(N, H, W, C, K, R, S, stride, pad, 0);
  if (kind == 2) {
    const int8_t* wp = nullptr;
    if (flags & NITI_CONV_FILTER_PREPARED) {
      wp = w;
    } else if (workspace != nullptr && aligned16(workspace) && workspace_bytes >= conv3x3_halo_filter_bytes(C, K)) {
      st = launch_halo_filter_prepare(w, static_cast<int8_t*>(workspace), K, C, 0, s);
      if (st != NITI_OK) return st;
      wp = static_cast<const int8_t*>(workspace);
    }
    if (wp != nullptr) return launch_conv3x3_halo(x, wp, y, N, H, C, K, flags, absmax, s);
  } else if (flags & NITI_CONV_FILTER_PREPARED) {
    // no copy exists for this shape: filter_prepare wrote nothing, so `w` must be the filter itself
  }
  const int P = (H + 2 * pad - R) / stride + 1, Q = (W + 2 * pad - S) / stride + 1;
  ConvProblem p{x, w, y, absmax, N, H, W, C, K, R, S, stride, pad,
                static_cast<long long>(P) * Q * K, static_cast<long long>(Q) * K, K, 1, 1, flags};
  return launch_conv_igemm(p, s);
}

extern "C" int niti_conv2d_i8_dgrad(const int8_t* err, const int8_t* w, int32_t* dx, int N, int H, int W, int C, int K,
                                    int R, int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  clear_error();
  int st = check_conv_dims("conv_dgrad", N, H, W, C, K, R, S, stride, pad);
  if (st == NITI_OK)
    st = check_flags("conv_dgrad", flags, NITI_EPI_F32_ROUNDTRIP | NITI_CONV_FILTER_PREPARED | NITI_CONV_FILTER_FORWARD_COPY);
  if (st != NITI_OK) return st;
  if (err == nullptr || w == nullptr || dx == nullptr) return fail(NITI_ERR_INVALID_ARG, "conv_dgrad: null pointer");
  if (stride != 1 || R != S || pad > R - 1)
    return fail(NITI_ERR_UNSUPPORTED, "conv_dgrad: needs stride 1, square filter, pad <= R-1 (stride=%d R=%d S=%d pad=%d)", stride, R, S, pad);
  if (K % 16 != 0) return fail(NITI_ERR_UNSUPPORTED, "conv_dgrad: K=%d must be a multiple of 16", K);
  if (!aligned16(err) || !aligned16(dx)) return fail(NITI_ERR_INVALID_ARG, "conv_dgrad: pointers must be 16-byte aligned");
  st = check_forward_copy_flag("conv_dgrad", 1, flags, N, H, W, C, K, R, S, stride, pad);
  if (st != NITI_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int kind = filter_copy_kind(N, H, W, C, K, R, S, stride, pad, 1);
  const int8_t* wt = w;
  if (!(flags & NITI_CONV_FILTER_PREPARED)) {
    const size_t need = niti_conv2d_i8_filter_workspace(N, H, W, C, K, R, S, stride, pad, 1);
    if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
      return fail(NITI_ERR_WORKSPACE, "conv_dgrad: needs %zu workspace bytes (16-byte aligned), got %zu", need, workspace_bytes);
    st = kind == 3 ? launch_halo_filter_prepare(w, static_cast<int8_t*>(workspace), C, K, 1, s)
                   : launch_filter_flip_transpose(w, static_cast<int8_t*>(workspace), K, R, S, C, s);
    if (st != NITI_OK) return st;
    wt = static_cast<const int8_t*>(workspace);
  } else if (!aligned16(w)) {
    return fail(NITI_ERR_INVALID_ARG, "conv_dgrad: prepared filter must be 16-byte aligned");
  }
  const int P = H + 2 * pad - R + 1, Q = W + 2 * pad - S + 1;
  // fprop over the error map: "input" [N,P,Q,K], "filter" [C,R,S,K], padding R-1-pad -> [N,H,W,C]
  if (kind == 3) return launch_conv3x3_halo(err, wt, dx, N, P, K, C, flags, absmax, s);
  ConvProblem p{err, wt, dx, absmax, N, P, Q, K, C, R, S, 1, R - 1 - pad,
                static_cast<long long>(H) * W * C, static_cast<long long>(W) * C, C, 1, 1, flags};
  return launch_conv_igemm(p, s);
}

// ---- convolution + requantisation in one launch -------------------------------------------------------
// wall-clock ticks (100 MHz) a grid-wide wait may last; NITI_SYNC_TIMEOUT_MS overrides the 2 s default (a healthy
// wait lasts microseconds; the limit only matters when other work holds part of the device).  Fractions are allowed
// (0.00001 ms is one tick); 0 makes every wait give up after its first look, which tests of that path use.
long long niti::sync_spin_limit() {
  static std::once_flag once;
  static long long spin_limit = 0;
  std::call_once(once, [] {
    const char* e = getenv("NITI_SYNC_TIMEOUT_MS");
    const double ms = e != nullptr ? atof(e) : 2000.0;
    const double ticks = ms * 100000.0;
    spin_limit = ticks >= 1.0 ? static_cast<long long>(ticks) : (ms > 0.0 ? 1LL : 0LL);
  });
  return spin_limit;
}

// One word per device that every grid-wide wait of the library sets when it gives up.  The sync words of a launch
// carry the same flag (word 1), but they are the caller's and are zeroed again before the next step; this word stays
// set until niti_sync_timeouts clears it, so a driver can look once per epoch instead of once per launch.
namespace {
static __device__ uint32_t g_timeout_word;
uint32_t* g_timeout_ptr[kDeviceSlots] = {};
int g_timeout_dev[kDeviceSlots];
}  // namespace
uint32_t* niti::timeout_word() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  const int slot = device_slot();
  if (g_timeout_ptr[slot] == nullptr || g_timeout_dev[slot] != dev) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_timeout_word)) != hipSuccess || p == nullptr) return nullptr;
    g_timeout_ptr[slot] = static_cast<uint32_t*>(p);
    g_timeout_dev[slot] = dev;
  }
  return g_timeout_ptr[slot];
}

extern "C" int niti_sync_timeouts(uint32_t* flag_out, int clear, void* stream) {
  clear_error();
  if (flag_out == nullptr) return fail(NITI_ERR_INVALID_ARG, "sync_timeouts: null pointer");
  uint32_t* const word = timeout_word();
  if (word == nullptr) return fail(NITI_ERR_LAUNCH, "sync_timeouts: cannot find the device word");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (hipMemcpyAsync(flag_out, word, sizeof(uint32_t), hipMemcpyDeviceToHost, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
    return fail(NITI_ERR_LAUNCH, "sync_timeouts: %s", hipGetErrorString(hipGetLastError()));
  if (clear != 0 && *flag_out != 0u) return launch_fill_u32(word, 1, 0u, s);
  return NITI_OK;
}

static int fused_blocks(int N, int H, int W, int C, int K, int R, int S, int stride, int pad, int dgrad) {
  if (halo_off()) return 0;
  if (!dgrad) return conv3x3_halo_requant_blocks(N, H, W, C, K, R, S, stride, pad);
  if (stride != 1 || R != S || pad > R - 1) return 0;
  const int P = H + 2 * pad - R + 1, Q = W + 2 * pad - S + 1;
  return conv3x3_halo_requant_blocks(N, P, Q, K, C, R, S, 1, R - 1 - pad);
}

extern "C" size_t niti_conv2d_i8_requant_sync_words(int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                                                    int dgrad) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || stride <= 0 || pad < 0) return 0;
  const int nb = fused_blocks(N, H, W, C, K, R, S, stride, pad, dgrad);
  return nb > 0 ? conv3x3_halo_sync_words(nb) : 0;
}

static int conv_requant(const char* who, int dgrad, const int8_t* x, const int8_t* w, int8_t* y8, int N, int H, int W, int C,
                        int K, int R, int S, int stride, int pad, unsigned flags, int target_bits, int method, int div_mode,
                        int bw_mode, unsigned rq_flags, const int8_t* relu_mask, uint32_t* sync, size_t sync_words,
                        int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* workspace,
                        size_t workspace_bytes, void* stream, int8_t* pool_out = nullptr, const int8_t* pool_x = nullptr,
                        int ties = -1, const int32_t* rand = nullptr) {
  clear_error();
  int st = check_conv_dims(who, N, H, W, C, K, R, S, stride, pad);
  if (st == NITI_OK)
    st = check_flags(who, flags, NITI_EPI_F32_ROUNDTRIP | NITI_CONV_FILTER_PREPARED | (dgrad ? NITI_CONV_FILTER_FORWARD_COPY : 0u));
  if (st != NITI_OK) return st;
  if (x == nullptr || w == nullptr || y8 == nullptr || sync == nullptr) return fail(NITI_ERR_INVALID_ARG, "%s: null pointer", who);
  if (!aligned16(x) || !aligned16(w) || !aligned16(y8)) return fail(NITI_ERR_INVALID_ARG, "%s: pointers must be 16-byte aligned", who);
  if (target_bits < 1 || target_bits > 7) return fail(NITI_ERR_INVALID_ARG, "%s: target_bits=%d outside 1..7", who, target_bits);
  if (method != NITI_ROUND_NEAREST && method != NITI_ROUND_PSEUDO_STOCHASTIC && !(method == NITI_ROUND_STOCHASTIC && rand != nullptr))
    return fail(NITI_ERR_UNSUPPORTED, "%s: rounding method %d needs random integers (the _sto entry points take them; or use the two-pass path)", who, method);
  if (rand != nullptr && !aligned16(rand)) return fail(NITI_ERR_INVALID_ARG, "%s: rand must be 16-byte aligned", who);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "%s: div_mode=%d", who, div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "%s: bw_mode=%d", who, bw_mode);
  if ((rq_flags & ~(NITI_RQ_RELU | NITI_RQ_SHIFT_HINT)) != 0u) return fail(NITI_ERR_INVALID_ARG, "%s: rq_flags=%#x", who, rq_flags);
  const int nb = fused_blocks(N, H, W, C, K, R, S, stride, pad, dgrad);
  if (nb == 0) return fail(NITI_ERR_UNSUPPORTED, "%s: shape not covered by the single-launch path; use the two-pass path", who);
  st = check_forward_copy_flag(who, dgrad, flags, N, H, W, C, K, R, S, stride, pad);
  if (st != NITI_OK) return st;
  if (sync_words < conv3x3_halo_sync_words(nb))
    return fail(NITI_ERR_WORKSPACE, "%s: needs %zu zeroed sync words, got %zu", who, conv3x3_halo_sync_words(nb), sync_words);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // geometry of the forward problem the kernel runs: the data gradient is a forward pass over the error map
  const int Hk = dgrad ? H + 2 * pad - R + 1 : H;
  const int Ck = dgrad ? K : C, Kk = dgrad ? C : K;
  const int8_t* wp = w;
  if (!(flags & NITI_CONV_FILTER_PREPARED)) {
    const size_t need = conv3x3_halo_filter_bytes(Ck, Kk);
    if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
      return fail(NITI_ERR_WORKSPACE, "%s: needs %zu workspace bytes (16-byte aligned), got %zu", who, need, workspace_bytes);
    st = launch_halo_filter_prepare(w, static_cast<int8_t*>(workspace), Kk, Ck, dgrad ? 1 : 0, s);
    if (st != NITI_OK) return st;
    wp = static_cast<const int8_t*>(workspace);
  }
  if (relu_mask != nullptr && !aligned16(relu_mask)) return fail(NITI_ERR_INVALID_ARG, "%s: relu_mask must be 16-byte aligned", who);
  if (pool_out != nullptr && (!aligned16(pool_out) || H % 2 != 0 || W % 2 != 0))
    return fail(NITI_ERR_INVALID_ARG, "%s: pool_out must be 16-byte aligned and the map side even", who);
  RequantSpec rq{target_bits, method, div_mode == NITI_DIV_TRUNC, bw_mode, rq_flags, sync_spin_limit(), timeout_word(), shift_out, exp_a, exp_b, exp_out, relu_mask,
                 pool_out};
  if (pool_x != nullptr) {   // y8 is the [N,2H,2W,C] result of the folded max-pool backward pass
    if (ties != NITI_TIES_FIRST && ties != NITI_TIES_ALL) return fail(NITI_ERR_INVALID_ARG, "%s: ties=%d", who, ties);
    if (relu_mask == nullptr || !aligned16(pool_x)) return fail(NITI_ERR_INVALID_ARG, "%s: pooled map and 16-byte aligned pooling input needed", who);
    rq.pool_x = pool_x;
    rq.unpool = y8;
    rq.ties_all = ties == NITI_TIES_ALL ? 1 : 0;
  }
  rq.rand = method == NITI_ROUND_STOCHASTIC ? rand : nullptr;
  return launch_conv3x3_halo_requant(x, wp, y8, N, Hk, Ck, Kk, flags, sync, rq, s);
}

extern "C" int niti_conv2d_i8_fprop_requant(const int8_t* x, const int8_t* w, int8_t* y8, int N, int H, int W, int C, int K,
                                            int R, int S, int stride, int pad, unsigned flags, int target_bits, int method,
                                            int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words,
                                            int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  return conv_requant("conv_fprop_requant", 0, x, w, y8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, method, div_mode,
                      bw_mode, rq_flags, nullptr, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace, workspace_bytes, stream);
}

extern "C" int niti_conv2d_i8_fprop_requant_pool(const int8_t* x, const int8_t* w, int8_t* y8, int8_t* pool_out, int N, int H, int W,
                                                 int C, int K, int R, int S, int stride, int pad, unsigned flags, int target_bits,
                                                 int method, int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync,
                                                 size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                                 int32_t* exp_out, void* workspace, size_t workspace_bytes, void* stream) {
  if (pool_out == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "conv_fprop_requant_pool: null pointer");
  }
  return conv_requant("conv_fprop_requant_pool", 0, x, w, y8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, method, div_mode,
                      bw_mode, rq_flags, nullptr, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace, workspace_bytes, stream,
                      pool_out);
}

extern "C" int niti_conv2d_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int N, int H, int W, int C, int K,
                                            int R, int S, int stride, int pad, unsigned flags, int target_bits, int method,
                                            int div_mode, int bw_mode, unsigned rq_flags, const int8_t* relu_mask, uint32_t* sync,
                                            size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                            int32_t* exp_out, void* workspace, size_t workspace_bytes, void* stream) {
  return conv_requant("conv_dgrad_requant", 1, err, w, dx8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, method, div_mode,
                      bw_mode, rq_flags, relu_mask, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace, workspace_bytes, stream);
}

extern "C" int niti_conv2d_i8_fprop_requant_sto(const int8_t* x, const int8_t* w, int8_t* y8, int8_t* pool_out, const int32_t* rand,
                                                int N, int H, int W, int C, int K, int R, int S, int stride, int pad, unsigned flags,
                                                int target_bits, int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync,
                                                size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                                int32_t* exp_out, void* workspace, size_t workspace_bytes, void* stream) {
  return conv_requant("conv_fprop_requant_sto", 0, x, w, y8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, NITI_ROUND_STOCHASTIC,
                      div_mode, bw_mode, rq_flags, nullptr, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace, workspace_bytes,
                      stream, pool_out, nullptr, -1, rand);
}

extern "C" int niti_conv2d_i8_dgrad_requant_sto(const int8_t* err, const int8_t* w, int8_t* dx8, const int32_t* rand, int N, int H, int W,
                                                int C, int K, int R, int S, int stride, int pad, unsigned flags, int target_bits,
                                                int div_mode, int bw_mode, unsigned rq_flags, const int8_t* relu_mask, uint32_t* sync,
                                                size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b,
                                                int32_t* exp_out, void* workspace, size_t workspace_bytes, void* stream) {
  return conv_requant("conv_dgrad_requant_sto", 1, err, w, dx8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, NITI_ROUND_STOCHASTIC,
                      div_mode, bw_mode, rq_flags, relu_mask, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace, workspace_bytes,
                      stream, nullptr, nullptr, -1, rand);
}

// ---- forward convolution + requantisation for callers that can neither allocate nor hand in scratch memory --------
// The sync words and the kernel-ready filter copy of niti_conv2d_i8_fprop_requant live in a device array of this
// library instead of caller memory.  Each GPU holds its own copy of the array at its own address, looked up once per
// device; host code only ever uses that address, never the array's name.
namespace {
constexpr size_t kStaticSyncWords = 16 + 4096 * static_cast<size_t>(NITI_SLOT_STRIDE);   // = conv3x3_halo_sync_words(4096)
constexpr size_t kStaticSyncBytes = (kStaticSyncWords * 4 + 255) / 256 * 256;
constexpr size_t kStaticFilterBytes = NITI_STATIC_FILTER_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticSyncBytes + kStaticFilterBytes];
unsigned char* g_scratch_ptr[kDeviceSlots] = {};
int g_scratch_dev[kDeviceSlots];

__global__ void copy_words_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

// address of this device's copy of `scratch` (nullptr + error message on failure)
unsigned char* static_scratch() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    fail(NITI_ERR_LAUNCH, "static scratch: no current device");
    return nullptr;
  }
  const int slot = device_slot();
  if (g_scratch_ptr[slot] == nullptr || g_scratch_dev[slot] != dev) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      fail(NITI_ERR_LAUNCH, "static scratch: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[slot] = static_cast<unsigned char*>(p);
    g_scratch_dev[slot] = dev;
  }
  return g_scratch_ptr[slot];
}
}  // namespace

extern "C" size_t niti_static_scratch_bytes(void) { return kStaticSyncBytes + kStaticFilterBytes; }

extern "C" int niti_conv2d_i8_fprop_requant_static(const int8_t* x, const int8_t* w, int8_t* y8, int N, int H, int W, int C, int K,
                                                   int R, int S, int stride, int pad, unsigned flags, int target_bits,
                                                   int method, int div_mode, int bw_mode, unsigned rq_flags, int32_t* shift_out,
                                                   const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                                   uint32_t* range_out, void* stream) {
  clear_error();
  const char* who = "conv_fprop_requant_static";
  int st = check_conv_dims(who, N, H, W, C, K, R, S, stride, pad);
  if (st != NITI_OK) return st;
  const int nb = fused_blocks(N, H, W, C, K, R, S, stride, pad, 0);
  if (nb == 0) return fail(NITI_ERR_UNSUPPORTED, "%s: shape not covered by the single-launch path", who);
  const size_t words = conv3x3_halo_sync_words(nb);
  if (words > kStaticSyncWords)
    return fail(NITI_ERR_UNSUPPORTED, "%s: %d workgroups need %zu sync words, the static scratch holds %zu", who, nb, words, kStaticSyncWords);
  const size_t fbytes = (flags & NITI_CONV_FILTER_PREPARED) ? 0 : conv3x3_halo_filter_bytes(C, K);
  if (fbytes > kStaticFilterBytes)
    return fail(NITI_ERR_UNSUPPORTED, "%s: the filter copy needs %zu bytes, the static scratch holds %zu (pass a prepared filter)", who,
                fbytes, kStaticFilterBytes);
  unsigned char* const base = static_scratch();
  if (base == nullptr) return NITI_ERR_LAUNCH;
  uint32_t* const sync = reinterpret_cast<uint32_t*>(base);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the array keeps the previous call's slots: clear them with a kernel (a memset node misbehaves in replayed graphs)
  st = launch_fill_u32(sync, static_cast<int64_t>(words), 0u, s);
  if (st != NITI_OK) return st;
  st = conv_requant(who, 0, x, w, y8, N, H, W, C, K, R, S, stride, pad, flags, target_bits, method, div_mode, bw_mode, rq_flags, nullptr,
                    sync, words, shift_out, exp_a, exp_b, exp_out, base + kStaticSyncBytes, kStaticFilterBytes, stream);
  if (st != NITI_OK || range_out == nullptr) return st;
  hipLaunchKernelGGL(copy_words_kernel, dim3(1), dim3(64), 0, s, sync, range_out, 2);
  return check_launch(who);
}

extern "C" int niti_conv2d_i8_dgrad_requant_unpool(const int8_t* err, const int8_t* w, int8_t* dx8_unpooled, const int8_t* pooled,
                                                   const int8_t* pool_in, int ties, int N, int H, int W, int C, int K, int R, int S,
                                                   int stride, int pad, unsigned flags, int target_bits, int method, int div_mode,
                                                   int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words,
                                                   int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                                   void* workspace, size_t workspace_bytes, void* stream) {
  if (pooled == nullptr || pool_in == nullptr) {
    clear_error();
    return fail(NITI_ERR_INVALID_ARG, "conv_dgrad_requant_unpool: null pointer");
  }
  return conv_requant("conv_dgrad_requant_unpool", 1, err, w, dx8_unpooled, N, H, W, C, K, R, S, stride, pad, flags, target_bits, method,
                      div_mode, bw_mode, rq_flags, pooled, sync, sync_words, shift_out, exp_a, exp_b, exp_out, workspace,
                      workspace_bytes, stream, nullptr, pool_in, ties);
}

extern "C" size_t niti_conv2d_i8_wgrad_workspace(int N, int H, int W, int C, int K, int R, int S, int pad) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || pad < 0) return 0;
  const int P = H + 2 * pad - R + 1, Q = W + 2 * pad - S + 1;
  if (P <= 0 || Q <= 0) return 0;
  if (wgrad3x3_supported(N, H, W, C, K, R, S, 1, pad)) return round256(wgrad3x3_workspace(N, H, C, K));
  const size_t np = static_cast<size_t>(round16(N));
  return round256(static_cast<size_t>(C) * H * W * np) + round256(static_cast<size_t>(K) * P * Q * np);
}

extern "C" int niti_conv2d_i8_wgrad(const int8_t* act, const int8_t* err, int32_t* dw, int N, int H, int W, int C, int K,
                                    int R, int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  clear_error();
  int st = check_conv_dims("conv_wgrad", N, H, W, C, K, R, S, stride, pad);
  if (st == NITI_OK) st = check_flags("conv_wgrad", flags, NITI_EPI_F32_ROUNDTRIP);
  if (st != NITI_OK) return st;
  if (act == nullptr || err == nullptr || dw == nullptr) return fail(NITI_ERR_INVALID_ARG, "conv_wgrad: null pointer");
  if (stride != 1) return fail(NITI_ERR_UNSUPPORTED, "conv_wgrad: stride %d (only 1)", stride);
  const size_t need = niti_conv2d_i8_wgrad_workspace(N, H, W, C, K, R, S, pad);
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(NITI_ERR_WORKSPACE, "conv_wgrad: needs %zu workspace bytes (16-byte aligned), got %zu", need, workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (wgrad3x3_supported(N, H, W, C, K, R, S, stride, pad)) {
    if (!aligned16(act) || !aligned16(err) || !aligned16(dw))
      return fail(NITI_ERR_INVALID_ARG, "conv_wgrad: pointers must be 16-byte aligned");
    return launch_wgrad3x3(act, err, dw, N, H, C, K, (flags & NITI_EPI_F32_ROUNDTRIP) != 0, absmax, workspace, s);
  }
  const int P = H + 2 * pad - R + 1, Q = W + 2 * pad - S + 1;
  const int np = round16(N);
  int8_t* act_t = static_cast<int8_t*>(workspace);                                 // [C][H*W][np]
  int8_t* err_t = act_t + round256(static_cast<size_t>(C) * H * W * np);           // [K][P*Q][np]
  st = launch_transpose_outer_inner_i8(act, act_t, N, H * W, C, np, s);
  if (st != NITI_OK) return st;
  st = launch_transpose_outer_inner_i8(err, err_t, N, P * Q, K, np, s);
  if (st != NITI_OK) return st;
  const int64_t nout = static_cast<int64_t>(K) * R * S * C;
  st = launch_fill_u32(reinterpret_cast<uint32_t*>(dw), nout, 0u, s);
  if (st != NITI_OK) return st;
  // The batch index becomes the reduction ("channel") index: images = C, filters = K, the
  // error map plays the filter window; output (c, r, s, k) is scattered to dw[k][r][s][c].
  const long long tiles = ((static_cast<long long>(C) * R * S + 127) / 128) * ((K + 127) / 128);
  const long long kg = static_cast<long long>(P) * Q * np;
  const int kiters = static_cast<int>((kg + 63) / 64);
  int split = pick_split(tiles, kiters);
  if (split < 2) split = 2;  // the scatter store path is the split-k one
  ConvProblem p{act_t, err_t, dw, nullptr, C, H, W, np, K, P, Q, 1, pad,
                1, static_cast<long long>(S) * C, C, static_cast<long long>(R) * S * C, split, 0u};
  st = launch_conv_igemm(p, s);
  if (st != NITI_OK) return st;
  return launch_post_i32(dw, nout, (flags & NITI_EPI_F32_ROUNDTRIP) != 0, absmax, s);
}

extern "C" size_t niti_conv2d_i8_wgrad_update_sync_words(int N, int H, int W, int C, int K, int R, int S, int stride, int pad) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || stride <= 0 || pad < 0) return 0;
  if (!wgrad3x3_supported(N, H, W, C, K, R, S, stride, pad) && !wgrad_small_shape(N, H, W, C, K, R, S, stride, pad)) return 0;
  const int nb = wgrad3x3_finish_blocks(C, K);
  return nb > 0 ? wgrad3x3_sync_words(nb) + wgrad_first_extra_words(H, C, K) : 0;
}

extern "C" int niti_conv2d_i8_wgrad_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int H, int W,
                                           int C, int K, int R, int S, int stride, int pad, unsigned flags, int mu, int method,
                                           int div_mode, int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out,
                                           int32_t* dw_out, int8_t* w_prepared, int32_t* shift_out, const int32_t* exp_a,
                                           const int32_t* exp_b, int32_t* exp_out, void* workspace, size_t workspace_bytes,
                                           void* stream) {
  clear_error();
  int st = check_conv_dims("conv_wgrad_update", N, H, W, C, K, R, S, stride, pad);
  if (st == NITI_OK) st = check_flags("conv_wgrad_update", flags, NITI_EPI_F32_ROUNDTRIP | NITI_CONV_SHIFT_HINT);
  if (st != NITI_OK) return st;
  if (act == nullptr || err == nullptr || w == nullptr || sync == nullptr)
    return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: null pointer");
  if (w_channels < 1 || w_channels > C) return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: w_channels=%d outside 1..C=%d", w_channels, C);
  if (mu < 1 || mu > 7) return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: mu=%d outside 1..7", mu);
  if (method != NITI_ROUND_NEAREST && method != NITI_ROUND_PSEUDO_STOCHASTIC)
    return fail(NITI_ERR_UNSUPPORTED, "conv_wgrad_update: rounding method %d needs random input; use the two-pass path", method);
  if (div_mode != NITI_DIV_FLOOR && div_mode != NITI_DIV_TRUNC) return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: div_mode=%d", div_mode);
  if (bw_mode != NITI_BW_INT && bw_mode != NITI_BW_F32) return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: bw_mode=%d", bw_mode);
  const size_t words = niti_conv2d_i8_wgrad_update_sync_words(N, H, W, C, K, R, S, stride, pad);
  if (words == 0) return fail(NITI_ERR_UNSUPPORTED, "conv_wgrad_update: shape not covered by the single-pass path; use the two-pass path");
  if (sync_words < words) return fail(NITI_ERR_WORKSPACE, "conv_wgrad_update: needs %zu zeroed sync words, got %zu", words, sync_words);
  const size_t need = niti_conv2d_i8_wgrad_workspace(N, H, W, C, K, R, S, pad);
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(NITI_ERR_WORKSPACE, "conv_wgrad_update: needs %zu workspace bytes (16-byte aligned), got %zu", need, workspace_bytes);
  if (!aligned16(act) || !aligned16(err) || (dw_out != nullptr && !aligned16(dw_out)))
    return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: act, err and dw_out must be 16-byte aligned");
  if (w_channels == C && (reinterpret_cast<uintptr_t>(w) % 4 != 0 || (g8_out != nullptr && reinterpret_cast<uintptr_t>(g8_out) % 4 != 0)))
    return fail(NITI_ERR_INVALID_ARG, "conv_wgrad_update: w and g8_out must be 4-byte aligned");
  if (w_prepared != nullptr && (filter_copy_kind(N, H, W, C, K, R, S, stride, pad, 0) != 2 || reinterpret_cast<uintptr_t>(w_prepared) % 4 != 0))
    return fail(NITI_ERR_UNSUPPORTED, "conv_wgrad_update: w_prepared needs a shape whose forward pass uses a kernel-ready filter copy, 4-byte aligned");
  RequantSpec rq{mu, method, div_mode == NITI_DIV_TRUNC, bw_mode, (flags & NITI_CONV_SHIFT_HINT) ? NITI_RQ_SHIFT_HINT : 0u, sync_spin_limit(),
                 timeout_word(), shift_out, exp_a, exp_b, exp_out, nullptr, nullptr};
  return launch_wgrad3x3_update(act, err, w, w_channels, N, H, C, K, (flags & NITI_EPI_F32_ROUNDTRIP) != 0, sync, rq, g8_out,
                                dw_out, w_prepared, workspace, static_cast<hipStream_t>(stream));
}

extern "C" size_t niti_gemm_i8_workspace(int trans_a, int trans_b, int m, int n, int k) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  if (gemm_kmajor_shape(trans_a, trans_b, m, n, k)) return gemm_kmajor_workspace(trans_a, trans_b, m, n, k);   // read as stored; partial sums of a split reduction
  const size_t kp = static_cast<size_t>(round16(k));
  size_t bytes = 0;
  if (trans_a || k % 16 != 0) bytes += round256(static_cast<size_t>(m) * kp);
  if (!trans_b || k % 16 != 0) bytes += round256(static_cast<size_t>(n) * kp);
  return bytes;
}

extern "C" int niti_gemm_i8(int trans_a, int trans_b, const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k,
                            unsigned flags, uint32_t* absmax, void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  if (m <= 0 || n <= 0 || k <= 0) return fail(NITI_ERR_INVALID_ARG, "gemm: non-positive extent (m=%d n=%d k=%d)", m, n, k);
  if (check_flags("gemm", flags, NITI_EPI_F32_ROUNDTRIP) != NITI_OK) return NITI_ERR_INVALID_ARG;
  if (a == nullptr || b == nullptr || c == nullptr) return fail(NITI_ERR_INVALID_ARG, "gemm: null pointer");
  if (!aligned16(c)) return fail(NITI_ERR_INVALID_ARG, "gemm: output must be 16-byte aligned");
  const size_t need = niti_gemm_i8_workspace(trans_a, trans_b, m, n, k);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need || !aligned16(workspace)))
    return fail(NITI_ERR_WORKSPACE, "gemm: needs %zu workspace bytes (16-byte aligned), got %zu", need, workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // reduction index slow in b (and in a): one launch, both operands read as stored
  if (gemm_kmajor_shape(trans_a, trans_b, m, n, k)) {
    if (!aligned16(a) || !aligned16(b)) return fail(NITI_ERR_INVALID_ARG, "gemm: operands must be 16-byte aligned");
    return launch_gemm_kmajor(trans_a, trans_b, a, b, c, m, n, k, (flags & NITI_EPI_F32_ROUNDTRIP) != 0, absmax, workspace, s);
  }
  const int kp = round16(k);
  int8_t* ws = static_cast<int8_t*>(workspace);
  const int8_t* a_use = a;  // [m][kp]
  const int8_t* b_use = b;  // [n][kp]
  int st;
  if (trans_a) {
    st = launch_transpose_outer_inner_i8(a, ws, k, 1, m, kp, s);  // [k][m] -> [m][kp]
    if (st != NITI_OK) return st;
    a_use = ws;
    ws += round256(static_cast<size_t>(m) * kp);
  } else if (kp != k) {
    hipLaunchKernelGGL(pad_rows_i8_kernel, dim3(1024), dim3(256), 0, s, a, ws, static_cast<int64_t>(m), k, kp);
    if ((st = check_launch("pad_rows")) != NITI_OK) return st;
    a_use = ws;
    ws += round256(static_cast<size_t>(m) * kp);
  }
  if (!trans_b) {
    st = launch_transpose_outer_inner_i8(b, ws, k, 1, n, kp, s);  // [k][n] -> [n][kp]
    if (st != NITI_OK) return st;
    b_use = ws;
  } else if (kp != k) {
    hipLaunchKernelGGL(pad_rows_i8_kernel, dim3(1024), dim3(256), 0, s, b, ws, static_cast<int64_t>(n), k, kp);
    if ((st = check_launch("pad_rows")) != NITI_OK) return st;
    b_use = ws;
  }
  if (!aligned16(a_use) || !aligned16(b_use)) return fail(NITI_ERR_INVALID_ARG, "gemm: operands must be 16-byte aligned");
  // a 1x1 convolution over an m x 1 x 1 "image" with kp channels and n filters
  ConvProblem p{a_use, b_use, c, absmax, m, 1, 1, kp, n, 1, 1, 1, 0, n, n, n, 1, 1, flags};
  // few output tiles and a long reduction (a fully connected layer on a batch): split the reduction over
  // workgroups that add into the zeroed output (integer addition: any split gives the same bits), then one
  // pass for the range
  const long long tiles = static_cast<long long>((m + 127) / 128) * ((n + 127) / 128);
  const int split = tiles >= 128 ? 1 : pick_split(tiles, (kp + 63) / 64);
  if (split > 1) {
    const int64_t nout = static_cast<int64_t>(m) * n;
    if ((st = launch_fill_u32(reinterpret_cast<uint32_t*>(c), nout, 0u, s)) != NITI_OK) return st;
    p.absmax = nullptr;
    p.split_k = split;
    if ((st = launch_conv_igemm(p, s)) != NITI_OK) return st;
    if (absmax == nullptr && !(flags & NITI_EPI_F32_ROUNDTRIP)) return NITI_OK;
    return launch_post_i32(c, nout, (flags & NITI_EPI_F32_ROUNDTRIP) != 0, absmax, s);
  }
  return launch_conv_igemm(p, s);
}
