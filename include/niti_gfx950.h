/*
 * libniti_gfx950 -- C ABI of the MI355X (gfx950) int8 training hot path of NITI.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream (passed as void*),
 * launches asynchronously on that stream and returns a status code (0 = success).  Nothing
 * here allocates device memory: outputs and workspaces are the caller's.  Layouts follow the
 * reference: activations NHWC int8, filters KRSC int8, conv results NPQK int32, GEMM
 * operands row-major.  "Reference" below is wangmaolin/niti; paths are relative to it.
 *
 * Per-tensor range: kernels that take `absmax` atomically max |value| into *absmax (uint32,
 * device memory, zeroed by the caller, e.g. with niti_fill_u32).  The requantisation kernels
 * read it back on the device, so no host synchronisation is needed between a GEMM and its
 * requantisation (the reference synchronises twice per tensor, ti_torch.py:369-377).
 */
#ifndef NITI_GFX950_H
#define NITI_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  NITI_OK = 0,
  NITI_ERR_INVALID_ARG = 1, /* null pointer, non-positive size, misaligned pointer */
  NITI_ERR_UNSUPPORTED = 2, /* shape outside what the kernels implement (message says which) */
  NITI_ERR_WORKSPACE = 3,   /* workspace missing or too small */
  NITI_ERR_LAUNCH = 4       /* HIP reported a launch error */
};

/* conv / gemm flags; a bit that the entry point called does not define is NITI_ERR_INVALID_ARG, not ignored */
#define NITI_EPI_F32_ROUNDTRIP 1u /* pass every int32 result through fp32 and back, as the
                                     reference's CUTLASS epilogue does
                                     (pytorch/cutlass-extension/cutlassconv_kernel.cu:78-85) */
#define NITI_CONV_FILTER_PREPARED 2u /* fprop / dgrad: `w` already is the kernel-ready filter copy written
                                        by niti_conv2d_i8_filter_prepare for the same shape; no workspace */
#define NITI_CONV_SHIFT_HINT 8u /* niti_conv2d_i8_wgrad_update only: *shift_out holds a predicted shift on entry, see
                                   NITI_RQ_SHIFT_HINT */
#define NITI_CONV_FILTER_FORWARD_COPY 4u /* data gradient only, with NITI_CONV_FILTER_PREPARED: `w` is the
                                            copy that niti_conv2d_i8_filter_prepare(.., dgrad = 0) made of
                                            the same filter (the one the forward pass reads) */
/* requant flags */
#define NITI_RQ_RELU 1u /* clamp the int8 result at 0 (TiReLU.forward, ti_torch.py:272-279) */
#define NITI_RQ_SHIFT_HINT 2u /* niti_conv2d_i8_*_requant: *shift_out holds a predicted shift on entry (the same
                                 tensor's shift of the previous training step).  The kernels store results before the
                                 tensor's range is final and store again if the shift turns out different; a good
                                 prediction saves that second pass.  The results do not depend on it. */

/* rounding method (ti_torch.py:23-69) / division meaning / bit-width evaluation / pool ties */
enum { NITI_ROUND_NEAREST = 0, NITI_ROUND_STOCHASTIC = 1, NITI_ROUND_PSEUDO_STOCHASTIC = 2 };
enum { NITI_DIV_FLOOR = 0, NITI_DIV_TRUNC = 1 };
enum { NITI_BW_INT = 0, NITI_BW_F32 = 1 };
enum { NITI_TIES_FIRST = 0, NITI_TIES_ALL = 1 };
#define NITI_POOL_BWD_RELU 2 /* or-ed into `ties` of niti_maxpool_i8_bwd: also zero dx where x <= 0, the backward pass
                                of a ReLU whose output is the pooling's input (TiReLU.backward, ti_torch.py:289) */

int niti_version(void);
const char* niti_status_string(int status);
/* message of the last failing call on this host thread ("" if none) */
const char* niti_last_error(void);

/* Host-side evaluation of the bit-width rule the kernels use (ti_torch.py:366-377):
 * NITI_BW_INT: ceil(log2(r)) as exact integer arithmetic; NITI_BW_F32: the reference's
 * int(ceil(log2f((float)r))) under a correctly rounded log2f.  r == 0 gives 0. */
int niti_bitwidth(uint32_t r, int bw_mode);

/*
 * Grid-wide waits that gave up.  Every single-launch kernel with a tensor-wide range (niti_conv2d_i8_*_requant,
 * niti_conv2d_i8_wgrad_update, niti_fc_i8_*) flags a wait that ran into its time limit in word 1 of its own sync words
 * AND in one word per device inside the library, which stays set until cleared here - so a driver whose sync words are
 * zeroed again every step can look once per epoch, and before it writes a checkpoint.  Copies that word to *flag_out
 * (host memory) after everything queued on `stream` so far has run (the call blocks), and zeroes it if clear != 0.
 * Non-zero means: some output since the last clear is invalid (other work kept part of the device busy).
 * No counterpart in the reference (its launches never wait for each other).
 */
int niti_sync_timeouts(uint32_t* flag_out, int clear, void* stream);

/* dst[0..n) = value */
int niti_fill_u32(uint32_t* dst, int64_t n, uint32_t value, void* stream);

/*
 * Kernel-ready filter copies.  The convolution kernels stream the filter in an arrangement of
 * their own (tap-major blocks for the 3x3 kernel that keeps activation rows resident in LDS,
 * flipped and transposed taps for the data gradient).  fprop / dgrad build that copy into the
 * caller's workspace on every call; a caller that reuses a filter (or wants the copy off the
 * critical path) can build it once with niti_conv2d_i8_filter_prepare and pass it in place of
 * `w` with NITI_CONV_FILTER_PREPARED.  Shape arguments are those of the convolution the copy
 * is for (w is always the layer's [K,R,S,C] filter; dgrad != 0 selects the data-gradient copy).
 * niti_conv2d_i8_filter_workspace returns the bytes needed (0: the kernels read w as stored).
 */
size_t niti_conv2d_i8_filter_workspace(int N, int H, int W, int C, int K, int R, int S, int stride, int pad, int dgrad);
int niti_conv2d_i8_filter_prepare(const int8_t* w, int8_t* dst, size_t dst_bytes, int N, int H, int W, int C, int K,
                                  int R, int S, int stride, int pad, int dgrad, void* stream);

/*
 * Convolution forward (cross-correlation), replaces cutlassconv_cuda.sp_conv and
 * .sp_conv_optimized (pytorch/cutlass-extension/cutlassconv.cpp:57-73,
 * cutlassconv_kernel.cu:38-319):
 *   y[n,p,q,k] = sum_{r,s,c} x[n, p*stride-pad+r, q*stride-pad+s, c] * w[k,r,s,c]
 * x: [N,H,W,C] int8, w: [K,R,S,C] int8, y: [N,P,Q,K] int32, P=(H+2*pad-R)/stride+1.
 * Requires C % 16 == 0 (the reference pads C the same way, ti_torch.py:178-183) and 16-byte
 * aligned x, w, y.  absmax may be NULL.  workspace: niti_conv2d_i8_filter_workspace(.., 0) bytes;
 * may be NULL / too small, then the kernel that reads w as stored is used.
 */
int niti_conv2d_i8_fprop(const int8_t* x, const int8_t* w, int32_t* y, int N, int H, int W, int C, int K, int R,
                         int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * Data gradient, replaces the reference's fprop-on-flipped-weights rewrite
 * (TiConv2d.backward, ti_torch.py:403-405):
 *   dx[n,h,w,c] = sum_{r,s,k} err[n, h+pad-r, w+pad-s, k] * w[k,r,s,c]
 * err: [N,P,Q,K] int8, w: [K,R,S,C] int8, dx: [N,H,W,C] int32.  Stride 1 and R == S only (the
 * reference's rewrite additionally needs 2*pad == R-1; here any pad <= R-1); needs K % 16 == 0.
 * Workspace: niti_conv2d_i8_filter_workspace(.., 1) bytes (the flipped / transposed filter copy,
 * which the reference materialises with flip/transpose/contiguous, ti_torch.py:404).
 */
int niti_conv2d_i8_dgrad(const int8_t* err, const int8_t* w, int32_t* dx, int N, int H, int W, int C, int K, int R,
                         int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * Convolution and requantisation in one launch.  Replaces the pairs
 *   cutlassconv_cuda.sp_conv_optimized + act_calc   (TiConv2d.forward,  ti_torch.py:393-397 with 103-117)
 *   cutlassconv_cuda.sp_conv_optimized + err_calc   (TiConv2d.backward, ti_torch.py:403-407 with 119-133)
 * with the same result as niti_conv2d_i8_fprop / _dgrad followed by niti_requant_i32_i8, bit for bit,
 * but the int32 sums stay in registers: every workgroup publishes the largest magnitude of its tile,
 * waits for all others, derives the tensor-wide shift and stores int8.
 *
 * Covered: 3x3, stride 1, pad 1, square inputs of side 2, 4, 8, 16 or 32, N*H*W % 256 == 0 (side 2: any N), input
 * channels % 16 == 0, output channels % 16 == 0, rounding NITI_ROUND_NEAREST or NITI_ROUND_PSEUDO_STOCHASTIC, and a
 * launch of at most 4096 workgroups (N*H*W/256 x ceil(out channels/128 or 64); side 2: ceil(N/32) x ceil(out
 * channels/32), which must fit on the device at once).  Launches of the other sides that do not fit on the device at
 * once run as two launches that do not wait (the second one settles tiles stored with another shift than the final
 * one).  niti_conv2d_i8_requant_sync_words returns 0 for shapes outside that (then use the two-pass entry points); the
 * entry points return NITI_ERR_UNSUPPORTED for them.
 *
 * sync: niti_conv2d_i8_requant_sync_words(...) uint32 words that are ZERO on entry (niti_fill_u32).  On return
 * word 0 holds max |sum| over the tensor; word 1 is non-zero if the wait for the other workgroups ran into its
 * time limit (2 s, or NITI_SYNC_TIMEOUT_MS from the environment), in which case the output is invalid - this
 * can only happen when other work keeps part of the device busy that long.  Launches that share a sync buffer
 * must not overlap.
 * flags: NITI_EPI_F32_ROUNDTRIP, NITI_CONV_FILTER_PREPARED (w is a copy made by niti_conv2d_i8_filter_prepare;
 * otherwise workspace must hold niti_conv2d_i8_filter_workspace bytes).  rq_flags: NITI_RQ_RELU, NITI_RQ_SHIFT_HINT.
 * shift_out / exp_a / exp_b / exp_out as in niti_requant_i32_i8 (each may be NULL).
 * relu_mask (data gradient only, may be NULL): int8 [N,H,W,C] like dx8; elements whose mask byte is not positive
 * are stored as zero AFTER the range and the rounding were taken from the unmasked sums.  Passing the layer's
 * own input activations folds in the backward pass of a ReLU that precedes the layer (TiReLU.backward,
 * ti_torch.py:284-290) - also across a max-pool in between, whose backward routes gradients only to positions
 * equal to the pooled maximum.
 */
size_t niti_conv2d_i8_requant_sync_words(int N, int H, int W, int C, int K, int R, int S, int stride, int pad, int dgrad);
int niti_conv2d_i8_fprop_requant(const int8_t* x, const int8_t* w, int8_t* y8, int N, int H, int W, int C, int K, int R,
                                 int S, int stride, int pad, unsigned flags, int target_bits, int method, int div_mode,
                                 int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words, int32_t* shift_out,
                                 const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* workspace,
                                 size_t workspace_bytes, void* stream);
/*
 * niti_conv2d_i8_fprop_requant that also writes the 2x2 / stride-2 maximum of its output: the TiMaxpool2d.forward ->
 * int8pool_cuda.int8_pool call that follows the layer (and its ReLU) in the reference's networks (ti_torch.py:302-307,
 * int8pool_kernel.cu:28-80; ti_vgg.py:28-35), taken from the rounded values before they leave the kernel.
 * pool_out: [N,H/2,W/2,K] int8, 16-byte aligned.  Same coverage as niti_conv2d_i8_fprop_requant.
 */
int niti_conv2d_i8_fprop_requant_pool(const int8_t* x, const int8_t* w, int8_t* y8, int8_t* pool_out, int N, int H, int W, int C,
                                      int K, int R, int S, int stride, int pad, unsigned flags, int target_bits, int method,
                                      int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words,
                                      int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                      void* workspace, size_t workspace_bytes, void* stream);
int niti_conv2d_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int N, int H, int W, int C, int K, int R,
                                 int S, int stride, int pad, unsigned flags, int target_bits, int method, int div_mode,
                                 int bw_mode, unsigned rq_flags, const int8_t* relu_mask, uint32_t* sync, size_t sync_words,
                                 int32_t* shift_out,
                                 const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* workspace,
                                 size_t workspace_bytes, void* stream);

/*
 * niti_conv2d_i8_dgrad_requant that also runs the backward pass of the 2x2 / stride-2 max-pool in front of the layer:
 * replaces TiConv2d.backward's data gradient + err_calc (ti_torch.py:403-407), the ReLU mask, and the
 * TiMaxpool2d.backward -> int8pool_cuda.int8_pool_backward call that follows it in the reference's networks
 * (ti_torch.py:309-316, int8pool_kernel.cu:82-138; ti_vgg.py:28-35), with the same result as
 * niti_conv2d_i8_dgrad_requant(.., relu_mask = pooled, ..) followed by niti_maxpool_i8_bwd(pooled, that, pool_in, .., 2, 2,
 * 0, ties).  N, H, W, C, K describe the convolution (H x W = the pooled map); pooled: [N,H,W,C] int8, the pooling's
 * output = the layer's input activations; pool_in: [N,2H,2W,C] int8, the pooling's input; dx8_unpooled: [N,2H,2W,C]
 * int8; all 16-byte aligned.  Elements whose pooled value is not positive get zero (the ReLU in front of the pooling);
 * the others go to the first position of their window that equals the pooled value (NITI_TIES_FIRST) or to all of them
 * (NITI_TIES_ALL).  Same coverage as niti_conv2d_i8_dgrad_requant.
 */
int niti_conv2d_i8_dgrad_requant_unpool(const int8_t* err, const int8_t* w, int8_t* dx8_unpooled, const int8_t* pooled,
                                        const int8_t* pool_in, int ties, int N, int H, int W, int C, int K, int R, int S, int stride,
                                        int pad, unsigned flags, int target_bits, int method, int div_mode, int bw_mode,
                                        unsigned rq_flags, uint32_t* sync, size_t sync_words, int32_t* shift_out,
                                        const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* workspace,
                                        size_t workspace_bytes, void* stream);

/*
 * The two single-launch entry points above with StoShift (ti_torch.py:33-46; selectable as ACT_ROUND_METHOD /
 * ERROR_ROUND_METHOD, ti_torch.py:460-463) folded in: rand holds one int32 per OUTPUT element, laid out like the
 * output ([N,H,W,K] forward, [N,H,W,C] data gradient), 16-byte aligned; it stands in for the reference's device
 * torch.randint(0, 2^shift) and only its low `shift` bits are used, so values drawn from any wider range work.  The
 * result equals niti_conv2d_i8_fprop / _dgrad followed by niti_requant_i32_i8(.., NITI_ROUND_STOCHASTIC, rand, ..).
 * pool_out (forward, may be NULL) as in niti_conv2d_i8_fprop_requant_pool.  Same coverage as the entry points above
 * except maps of side 2 (NITI_ERR_UNSUPPORTED: use the two-pass entry points there).
 */
int niti_conv2d_i8_fprop_requant_sto(const int8_t* x, const int8_t* w, int8_t* y8, int8_t* pool_out, const int32_t* rand, int N, int H,
                                     int W, int C, int K, int R, int S, int stride, int pad, unsigned flags, int target_bits,
                                     int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words,
                                     int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                     void* workspace, size_t workspace_bytes, void* stream);
int niti_conv2d_i8_dgrad_requant_sto(const int8_t* err, const int8_t* w, int8_t* dx8, const int32_t* rand, int N, int H, int W, int C,
                                     int K, int R, int S, int stride, int pad, unsigned flags, int target_bits, int div_mode,
                                     int bw_mode, unsigned rq_flags, const int8_t* relu_mask, uint32_t* sync, size_t sync_words,
                                     int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                     void* workspace, size_t workspace_bytes, void* stream);

/*
 * niti_conv2d_i8_fprop_requant for callers that cannot allocate device memory or hand in scratch memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arithmetic and the same results as niti_conv2d_i8_fprop_requant; the sync words and the kernel-ready filter copy live
 * in a device array inside the library (niti_static_scratch_bytes() bytes per GPU the library runs on, about 4.1 MiB,
 * held until the process ends), which the call clears with a small kernel before use.  It calls no hipMalloc / hipFree
 * and nothing that allocates.
 * Limits: a launch of at most 4096 workgroups (as niti_conv2d_i8_fprop_requant) and a filter copy
 * (niti_conv2d_i8_filter_workspace(.., 0)) of at most 4 MiB unless NITI_CONV_FILTER_PREPARED is passed (then `w` is
 * the caller's prepared copy); beyond them the call returns NITI_ERR_UNSUPPORTED and launches nothing.
 * range_out (may be NULL): two words, [0] = max |sum| over the tensor, [1] != 0 if the wait for the other workgroups
 * ran into its time limit (what words 0 and 1 of `sync` hold after niti_conv2d_i8_fprop_requant).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two host threads) race.
 */
size_t niti_static_scratch_bytes(void);
int niti_conv2d_i8_fprop_requant_static(const int8_t* x, const int8_t* w, int8_t* y8, int N, int H, int W, int C, int K, int R,
                                        int S, int stride, int pad, unsigned flags, int target_bits, int method, int div_mode,
                                        int bw_mode, unsigned rq_flags, int32_t* shift_out, const int32_t* exp_a,
                                        const int32_t* exp_b, int32_t* exp_out, uint32_t* range_out, void* stream);

/*
 * Weight gradient, replaces the reference's fprop-on-transposed-operands rewrite
 * (ti_torch.py:430-432) and, for the first layer, conv2d_weight_int8 -> group_conv
 * (ti_torch.py:194-233):
 *   dw[k,r,s,c] = sum_{n,p,q} err[n,p,q,k] * act[n, p+r-pad, q+s-pad, c]
 * act: [N,H,W,C] int8, err: [N,P,Q,K] int8, dw: [K,R,S,C] int32.  Stride 1 only; any C, K, N.
 * Workspace: niti_conv2d_i8_wgrad_workspace() bytes.  absmax may be NULL.
 */
size_t niti_conv2d_i8_wgrad_workspace(int N, int H, int W, int C, int K, int R, int S, int pad);
int niti_conv2d_i8_wgrad(const int8_t* act, const int8_t* err, int32_t* dw, int N, int H, int W, int C, int K,
                         int R, int S, int stride, int pad, unsigned flags, uint32_t* absmax, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * Weight gradient, gradient rounding and weight update in one call.  Replaces the chain
 *   cutlassconv_cuda.sp_conv_optimized on transposed operands (ti_torch.py:430-432) -> grad_calc
 *   (ti_torch.py:135-147) -> UpdateWeight.weight_update (ti_torch.py:11-21)
 * with the same result as niti_conv2d_i8_wgrad followed by niti_grad_update_i8, bit for bit; the int32 gradient
 * is only written when dw_out is given.  The partial sums of the weight-gradient kernel are added up, the
 * tensor-wide range is exchanged between the workgroups that add them, and
 *   g = round(dw >> max(bitwidth(max|dw|) - mu, 0)),  w = clip(w - g, +-127).
 * Maps of side 8, 16 and 32 with N*H*W % 256 == 0 run all of it as one launch (its at most 256 workgroups add
 * their partial sums once all of them have arrived, so they must all be resident: nothing else may run on the
 * device beside it); other shapes, or a device that cannot hold the grid at once, run a main and a finishing launch.
 *
 * Covered: the shapes of the native 3x3 weight-gradient kernel (3x3, stride 1, pad 1, square maps of side 2, 4, 8,
 * 16 or 32, C % 16 == 0, K % 16 == 0, N*H*W % 128 == 0, even N for side 8, N*H*W % 256 == 0 for sides 2 and 4) with
 * K*9*C <= 4M, rounding
 * NITI_ROUND_NEAREST or NITI_ROUND_PSEUDO_STOCHASTIC.  niti_conv2d_i8_wgrad_update_sync_words returns 0 otherwise.
 * Two kinds of layer run as a single launch instead of the kernel pair: the first layer (side 32, C == 16 with
 * w_channels <= 3, K 32 / 64 / 128 / 256: a workgroup per image adds its sums with integer atomics into extra zeroed
 * sync words, the last workgroup to arrive rounds and updates - no workgroup waits for another) and layers on maps of
 * side 2 and 4 with C % 32 == 0, K % 32 == 0 and at most 8192 pixels (a workgroup owns 32 x 32 channels x 9 taps over
 * all pixels; for these any N is covered, not only N*H*W % 256 == 0).
 *
 * act: [N,H,W,C] int8 (C may include zero channel padding); err: [N,H,W,K] int8; w: [K,3,3,w_channels] int8,
 * updated in place, w_channels <= C (gradient columns beyond w_channels are padding and are dropped).
 * g8_out (optional): rounded gradient, laid out like w.  dw_out (optional): int32 gradient [K,3,3,C].
 * w_prepared (optional): the copy niti_conv2d_i8_filter_prepare(.., dgrad = 0) made of the filter [K,3,3,C] (w
 * zero-padded to C channels); the updated weights are written into it as well, so the next forward pass can run
 * with NITI_CONV_FILTER_PREPARED without a new copy.
 * sync: as for niti_conv2d_i8_fprop_requant (zero on entry; word 0 = max |dw|, word 1 = wait timed out).
 * workspace: niti_conv2d_i8_wgrad_workspace bytes.  flags: NITI_EPI_F32_ROUNDTRIP.
 */
size_t niti_conv2d_i8_wgrad_update_sync_words(int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
int niti_conv2d_i8_wgrad_update(const int8_t* act, const int8_t* err, int8_t* w, int w_channels, int N, int H, int W, int C,
                                int K, int R, int S, int stride, int pad, unsigned flags, int mu, int method, int div_mode,
                                int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* dw_out,
                                int8_t* w_prepared, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                                void* workspace, size_t workspace_bytes, void* stream);

/*
 * int8 x int8 -> exact int32 GEMM, replaces int8mm_cuda.int8_mm
 * (pytorch/int8mm-extension/int8mm.cpp:9-14, int8mm_kernel.cu:8-34):
 *   c[m,n] = sum_k opA[m,k] * opB[k,n],  c row-major with leading dimension n.
 * trans_a == 0: a is [m,k] row-major; 1: a is [k,m].  trans_b == 0: b is [k,n]; 1: b is [n,k].
 * Operands are read as stored, no operand copy: (trans_a=0, trans_b=1) with k % 16 == 0;
 * trans_b=0 - the form the reference's extension receives (trans_a=0) and the one with both
 * reduction indices slow (trans_a=1, m % 16 == 0) - with n % 32 == 0 and k % 32 == 0, through
 * transposing LDS reads; (trans_a=1, trans_b=1) with m % 32 == 0 and k % 32 == 0 the same way
 * (it fills the [n,m] buffer behind the transposed view that int8_mm returns, from lhs and rhs
 * as the reference passes them).  One launch - except that the forms with trans_a == trans_b
 * whose result has few tiles and whose reduction is long (n, k multiples of 128; in the doubly
 * transposed form m, k) split the reduction over workgroups: the int32 parts go to the workspace
 * and a second small launch adds them.  Other shapes first re-lay the operand(s) into the
 * workspace.  niti_gemm_i8_workspace() reports the bytes either way (0 when none are needed).
 */
size_t niti_gemm_i8_workspace(int trans_a, int trans_b, int m, int n, int k);
int niti_gemm_i8(int trans_a, int trans_b, const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k,
                 unsigned flags, uint32_t* absmax, void* workspace, size_t workspace_bytes, void* stream);

/* max |x[i]| atomically folded into *absmax (RangeEstimate, ti_torch.py:369-377) */
int niti_absmax_i32(const int32_t* x, int64_t n, uint32_t* absmax, void* stream);

/*
 * act_calc / err_calc / grad_calc (ti_torch.py:103-147) in one pass:
 *   shift = bitwidth(*absmax) - target_bits
 *   shift >= 1: y = clip(round_method(x, shift), +-127)   else: y = low byte of x (128 wraps)
 *   *shift_out = max(shift, 0)                            (shift_out may be NULL)
 *   *exp_out   = max(shift, 0) + *exp_a + *exp_b          (each of the three may be NULL)
 * The last line is the exponent bookkeeping the reference does on the host: exp_in + shift
 * with exp_in = act_in_exp + weight_exp (ti_torch.py:111,396), err_exp + weight_exp + shift
 * (ti_torch.py:261,407), err_exp + grad_shift + act_in_exp (ti_torch.py:20).
 * target_bits = 7 for activations and errors, GRAD_BITWIDTH (5/4/3) for gradients.
 * rand: one int32 per element, NITI_ROUND_STOCHASTIC only (stands in for the reference's device
 * torch.randint(0, 2^shift), ti_torch.py:41); only the low `shift` bits are used, so values
 * already in [0, 2^shift) are taken as they are and wider uniform bits may be supplied when the
 * host does not know the shift.
 */
int niti_requant_i32_i8(const int32_t* x, int8_t* y, int64_t n, const uint32_t* absmax, int target_bits,
                        int method, int div_mode, int bw_mode, const int32_t* rand, unsigned flags,
                        int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                        void* stream);

/*
 * UpdateWeight.weight_update (ti_torch.py:16-21) fused with grad_calc:
 *   g8 = grad_calc(g, mu);  w = clip(int16(w) - int16(g8), +-127)
 * g8_out (int8, may be NULL) receives the rounded gradient.
 */
int niti_grad_update_i8(const int32_t* g, int8_t* w, int64_t n, const uint32_t* absmax, int mu, int method,
                        int div_mode, int bw_mode, const int32_t* rand, int8_t* g8_out, int32_t* shift_out,
                        const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);

/* dst [rows][kpad] = src [rows][k] with zeros appended to every row: the zero padding of the channel dimension to a
   multiple of 16 that conv2d_int8 applies to input and filter (ti_torch.py:182-187), as one launch */
int niti_pad_rows_i8(const int8_t* src, int8_t* dst, int64_t rows, int k, int kpad, void* stream);

/* w = clip(int16(w) - int16(g), +-127)  (ti_torch.py:21) */
int niti_weight_update_i8(int8_t* w, const int8_t* g, int64_t n, void* stream);

/* y = max(x, 0) (ti_torch.py:278);  dx = act > 0 ? dy : 0 (ti_torch.py:289) */
int niti_relu_i8_fwd(const int8_t* x, int8_t* y, int64_t n, void* stream);
int niti_relu_i8_bwd(const int8_t* act, const int8_t* dy, int8_t* dx, int64_t n, void* stream);

/* TiFloatToInt8 (ti_torch.py:341-356) and the NCHW -> NHWC change that follows it (ti_net.py:19), two launches:
   r = max|x|, bw = ceil(log2 r), y = int8(clamp(round_half_even(x * 2^(bits - bw)), -128, 127)), *exp_out = bw - bits.
   x: float [N,C,H,W]; y: int8 [N,H,W,cpad] with channels C..cpad-1 zero (cpad % 4 == 0; 16 feeds the convolution kernels
   directly); absmax_bits: one ZEROED word that receives the bits of r.  An all-zero batch gives zeros and exponent 0
   (the reference's float sequence produces NaN there). */
int niti_quantize_f32_i8(const float* x, int8_t* y, int N, int C, int H, int W, int cpad, int bits, uint32_t* absmax_bits,
                         int32_t* exp_out, void* stream);

/* TiDropout (ti_torch.py:439-455): y[m][f] = x[m][f] * mask[f] with one keep (1) / drop (0) byte per feature, and - when
   exp_out is given - exp_out = exp_in + exp_add (the layer raises the exponent by one; exp_in NULL counts as 0), as one
   launch.  The backward pass is the same product on the error (exp_out NULL).  features % 16 == 0, 16-byte aligned. */
int niti_mask_features_i8(const int8_t* x, const int8_t* mask, int8_t* y, int64_t rows, int features, const int32_t* exp_in,
                          int32_t* exp_out, int exp_add, void* stream);

/*
 * NHWC int8 max pooling, replaces int8pool_cuda.int8_pool / int8_pool_backward
 * (pytorch/int8pool-extension/int8pool.cpp:37-57, int8pool_kernel.cu:28-138).
 * x: [N,H,W,C], y/dy: [N,P,Q,C], dx: [N,H,W,C], P=(H+2*pad-ks)/stride+1.
 * Backward routes dy to the position(s) of x equal to y: the first in (kh,kw) scan order
 * (NITI_TIES_FIRST) or all of them (NITI_TIES_ALL); overlapping windows add.  NITI_POOL_BWD_RELU or-ed into
 * `ties` folds the backward pass of a ReLU in front of the pooling into the same launch.
 */
int niti_maxpool_i8_fwd(const int8_t* x, int8_t* y, int N, int H, int W, int C, int ks, int stride, int pad,
                        void* stream);
int niti_maxpool_i8_bwd(const int8_t* y, const int8_t* dy, const int8_t* x, int8_t* dx, int N, int H, int W, int C,
                        int ks, int stride, int pad, int ties, void* stream);

/*
 * TiLinear with at most 16 output features (the classifier), each pass as one launch with its requantisation
 * folded in (ti_torch.py:241-266); operands as the layer stores them: act [M][F], w [O][F], err [M][O], int8.
 *   fwd_requant:   out8 [M][O] = act_calc(act * w^T)            (ti_torch.py:245-249)
 *   dgrad_requant: dx8 [M][F]  = err_calc(err * w)              (ti_torch.py:256-261)
 *   wgrad_update:  g = grad_calc(err^T * act), w = clip(w - g)  (ti_torch.py:263-265, 16-21); g8_out optional
 * `which` names the pass for the sync query, which returns 0 for shapes these kernels do not cover (then use
 * niti_gemm_i8 + niti_requant_i32_i8 / niti_grad_update_i8).  sync: zeroed uint32 words as for the convolutions
 * (word 0 range out, word 1 time-out flag, one slot per workgroup from word 16, four words apart).
 * Rounding NITI_ROUND_NEAREST or NITI_ROUND_PSEUDO_STOCHASTIC; shift_out / exp_* as in niti_requant_i32_i8.
 */
enum { NITI_FC_FORWARD = 0, NITI_FC_DGRAD = 1, NITI_FC_WGRAD = 2 };
size_t niti_fc_i8_sync_words(int which, int M, int O, int F);
int niti_fc_i8_fwd_requant(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int target_bits, int method,
                           int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync, size_t sync_words, int32_t* shift_out,
                           const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);
int niti_fc_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int M, int O, int F, int target_bits, int method,
                             int div_mode, int bw_mode, uint32_t* sync, size_t sync_words, int32_t* shift_out,
                             const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);
int niti_fc_i8_wgrad_update(const int8_t* err, const int8_t* act, int8_t* w, int M, int O, int F, int mu, int method,
                            int div_mode, int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* shift_out,
                            const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);

/*
 * TiLinear of any width (ti_torch.py:241-266) on the matrix cores, each pass as one launch with its requantisation
 * folded in; replaces int8mm_cuda.int8_mm (int8mm.cpp:9-14, int8mm_kernel.cu:8-34) + the transposing copies around it
 * (ti_torch.py:246,263,176) + act_calc / err_calc / grad_calc + weight_update.  Operands as the layer stores them:
 * act [M][F], w [O][F], err [M][O], int8; no operand is re-laid and no int32 product is written to memory.
 * Rounding: NITI_ROUND_NEAREST, NITI_ROUND_PSEUDO_STOCHASTIC, or NITI_ROUND_STOCHASTIC with `rand` (one int32 per
 * OUTPUT element - [M][O], [M][F], [O][F] - low `shift` bits used, as in niti_requant_i32_i8; NULL otherwise).
 * Shapes: forward F % 16 == 0, O % 4 == 0; dgrad O % 32 == 0, F % 32 == 0, O <= 4096; wgrad O % 16 == 0, F % 16 == 0;
 * 16-byte aligned operands.  niti_linear_i8_sync_words returns 0 for shapes outside that or whose workgroups the
 * current device does not hold at once (then use niti_gemm_i8 + niti_requant_i32_i8 / niti_grad_update_i8).
 * sync, shift_out, exp_* as in niti_fc_i8_*.
 */
size_t niti_linear_i8_sync_words(int which, int M, int O, int F);
int niti_linear_i8_fwd_requant(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int target_bits, int method,
                               int div_mode, int bw_mode, unsigned rq_flags, const int32_t* rand, uint32_t* sync, size_t sync_words,
                               int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);
int niti_linear_i8_dgrad_requant(const int8_t* err, const int8_t* w, int8_t* dx8, int M, int O, int F, int target_bits, int method,
                                 int div_mode, int bw_mode, const int32_t* rand, uint32_t* sync, size_t sync_words,
                                 int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);
int niti_linear_i8_wgrad_update(const int8_t* err, const int8_t* act, int8_t* w, int M, int O, int F, int mu, int method,
                                int div_mode, int bw_mode, const int32_t* rand, uint32_t* sync, size_t sync_words, int8_t* g8_out,
                                int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out, void* stream);

/*
 * Integer cross-entropy gradient, TiLoss.forward (ti_loss.py:5-36), as one launch: out_val [n][classes] int8 logits
 * with exponent *out_exp (device scalar), target [n] int64 class indices, rand [n][classes] int32 random integers
 * (the low four bits stand in for the reference's torch.randint(0, 16)) -> grad [n][classes] int8 with exponent 0.
 * Every float32 operation of the reference's sequence is kept in order (base-2 soft-max for out_exp > -7, the
 * quadratic 1 + x + x^2/2 form below), the int64 truncating sums included; the last step is StoShift(.., 4).
 */
int niti_loss_grad_i8(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, const int32_t* rand,
                      int8_t* grad, int n, int classes, int div_mode, void* stream);

/*
 * Random integers drawn inside the kernels.  The reference draws a dropout mask (ti_torch.py:444) and the random
 * integers of the loss gradient's StoShift (ti_loss.py:35, ti_torch.py:88-90) with torch.randint on the device, a
 * launch each; the entry points below that take `rng` draw them themselves.  rng: four uint32 words in device memory,
 * {key0, key1, step, 0}, which the caller initialises once (any key, step 0) and the kernels advance: every launch
 * that draws adds 1 to `step` when its last workgroup is done.  Word i of stream s in a launch that finds step t is
 * output word (i & 3) of Philox4x32-10 with counter {i >> 2, s, t, 0} and key {key0, key1} (stream 1: dropout, a
 * feature is kept when bit 0 of its word is set; stream 2: loss gradient, logit i uses the low four bits of word i).
 * niti_rng_words_u32 writes the first n words of a stream that a launch would draw in the state's present step (it
 * does not advance the state): what a test or a replaying host needs to predict a kernel's draws.
 * niti_loss_grad_i8_rng is niti_loss_grad_i8 with the random integers drawn from rng.
 */
int niti_rng_words_u32(const uint32_t* rng, uint32_t stream_id, uint32_t* out, size_t n, void* stream);
int niti_loss_grad_i8_rng(const int8_t* out_val, const int32_t* out_exp, const int64_t* target, uint32_t* rng, int8_t* grad,
                          int n, int classes, int div_mode, void* stream);

/*
 * The classifier at the end of a network in two launches: TiDropout.forward + TiLinear.forward (+ TiLoss.forward when
 * the targets are known), then TiLinear.backward + TiDropout.backward (ti_vgg.py:37-40, ti_torch.py:241-266, :439-455,
 * ti_loss.py:5-36; in the reference about sixty tensor-operation launches, with the passes above nine).
 * niti_head_i8_forward: out8 [M][O] = act_calc((act * mask) @ w^T) as niti_fc_i8_fwd_requant, with
 *   dropout 0: no mask; 1: drop_mask [F] (bytes 0 / 1) is read; 2: the mask is drawn from rng and written to drop_mask;
 *   exp_bias is added to *exp_out (TiDropout adds 1 to the exponent);
 *   target [M] int64 or null: with it loss_grad [M][O] receives what niti_loss_grad_i8 gives for the logits just
 *   written (their exponent being *exp_out), with loss_rand [M][O] or, when that is null, draws from rng.
 * niti_head_i8_backward: err [M][O] (exponent *exp_err) ->
 *   dx8 [M][F] = err_calc(err @ w) * mask, *err_exp_out = shift + *exp_err + *exp_w (ti_torch.py:258-260);
 *   w = clip(w - grad_calc(err^T @ (act * mask), grad_bits)) in place (ti_torch.py:262-263, :16-21), g8_out [O][F]
 *   optionally the rounded gradient, *grad_exp_out = its shift + *err_exp_out + *exp_act + exp_act_bias.
 *   act is the tensor in front of the dropout; drop_mask may be null.  M <= 256, O <= 16, F a multiple of 64.
 * Both need every workgroup resident (NITI_ERR_UNSUPPORTED otherwise) and zeroed sync words
 * (niti_head_i8_sync_words(backward, ...), 0 = shape not covered): word 0 range (backward: of the data gradient),
 * word 1 time-out flag, word 2 (backward) range of the weight gradient.  Rounding NITI_ROUND_NEAREST or
 * NITI_ROUND_PSEUDO_STOCHASTIC.
 */
size_t niti_head_i8_sync_words(int backward, int M, int O, int F);
int niti_head_i8_forward(const int8_t* act, const int8_t* w, int8_t* out8, int M, int O, int F, int dropout, int8_t* drop_mask,
                         uint32_t* rng, int exp_bias, const int64_t* target, const int32_t* loss_rand, int8_t* loss_grad,
                         int target_bits, int method, int div_mode, int bw_mode, unsigned rq_flags, uint32_t* sync,
                         size_t sync_words, int32_t* shift_out, const int32_t* exp_a, const int32_t* exp_b, int32_t* exp_out,
                         void* stream);
int niti_head_i8_backward(const int8_t* err, const int8_t* act, const int8_t* drop_mask, int8_t* w, int8_t* dx8, int M, int O,
                          int F, int err_bits, int err_method, int grad_bits, int grad_method, int div_mode, int bw_mode,
                          uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* err_shift_out, int32_t* grad_shift_out,
                          const int32_t* exp_err, const int32_t* exp_w, const int32_t* exp_act, int exp_act_bias,
                          int32_t* err_exp_out, int32_t* grad_exp_out, void* stream);
/*
 * niti_head_i8_backward with the backward pass of the 2 x 2 / stride-2 max-pool whose flattened output act is
 * (ti_vgg.py:33-37: TiMaxpool2d, TiFlat in front of the classifier; ti_torch.py:302-316, int8pool_kernel.cu:84-138):
 * act [M][P][Q][C] = maxpool(pool_in [M][2P][2Q][C]), F = P Q C, C a multiple of 64.  unpooled [M][2P][2Q][C] receives
 * what niti_maxpool_i8_bwd(act, dx8, pool_in, ...) would write, pool_flags = NITI_TIES_FIRST / NITI_TIES_ALL, optionally
 * | NITI_POOL_BWD_RELU.  dx8 may be null here (only the routed gradient is wanted).
 */
int niti_head_i8_backward_unpool(const int8_t* err, const int8_t* act, const int8_t* drop_mask, int8_t* w, int8_t* dx8, int M,
                                 int O, int F, int err_bits, int err_method, int grad_bits, int grad_method, int div_mode,
                                 int bw_mode, uint32_t* sync, size_t sync_words, int8_t* g8_out, int32_t* err_shift_out,
                                 int32_t* grad_shift_out, const int32_t* exp_err, const int32_t* exp_w, const int32_t* exp_act,
                                 int exp_act_bias, int32_t* err_exp_out, int32_t* grad_exp_out, const int8_t* pool_in,
                                 int8_t* unpooled, int P, int Q, int C, int pool_flags, void* stream);

/*
 * Grouped int8 convolution with float32 output, replaces int8conv_cuda.group_conv
 * (pytorch/int8conv-extension/int8conv.cpp:35-44, int8conv_kernel.cu:248-334):
 * x: [N,H,W,G*Cg] int8, w: [K,R,S,Cg] int8 (K % G == 0, filter k belongs to group k/(K/G)),
 * y: [N,P,Q,K] float32 (integer-valued; exact while |sum| < 2^24).
 */
int niti_group_conv_i8_f32(const int8_t* x, const int8_t* w, float* y, int N, int H, int W, int C, int K, int R,
                           int S, int Cg, int stride, int pad, int dilation, int groups, void* stream);

/* ==================================================================================================================
 * MEASUREMENT ONLY - not part of the boundary a reference checkout binds to; nothing in the layers calls it.
 * ================================================================================================================== */
/*
 * Measurement aid, no counterpart in the reference: a register-resident int8 MFMA loop (v_mfma_i32_32x32x32_i8, no LDS
 * and no memory traffic inside the loop) over operand fragments read once from `operands` (operand_bytes >= 128,
 * 16-byte aligned).  `workgroups` x 8 wavefronts each run `iters` rounds of 12 MFMAs = iters * 12 * 65536 int8
 * operations per wavefront.  The rate depends on the operand VALUES (the shader clock follows the multipliers' power
 * draw): time it with events for constant and for random operands to see the ceiling the convolution kernels run
 * under.  out: workgroups * 512 int32 checksums.  clocks (may be NULL): [0] shader clocks, [1] 100 MHz ticks that
 * workgroup 0 spent in the loop.
 */
int niti_mfma_probe_i8(const int8_t* operands, size_t operand_bytes, int workgroups, int iters, int32_t* out,
                       int64_t* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NITI_GFX950_H */
