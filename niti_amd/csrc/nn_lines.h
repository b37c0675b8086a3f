// Main loop shared by the whole-line kernels: 32 rows x 128 columns of c[m][n] = sum_k a[m][k] b[k][n] (a rows and
// b rows contiguous in memory, i.e. the reduction index is the slow one in b) over a range of the reduction, both
// operands staged through LDS one whole 128-byte line per row.
//
// The path from L2 into a compute unit moves whole lines at several times the rate of 32- or 64-byte pieces, so per
// chunk of 128 reduction steps the 512 threads stage b[k .. k+128)[n0 .. n0+128) (128 lines) and
// a[m0 .. m0+32)[k .. k+128) (32 lines) with buffer_load ... lds: an instruction moves eight rows' lines, lane ->
// (row lane / 8, 16-byte piece lane % 8), and writes them to LDS in lane order, so the XOR swizzle that keeps the
// fragment reads off each other's banks is applied to the address in memory.  A ring of three stages, one barrier per
// chunk.  8 wavefronts = 4 column quarters (ft) x 2 halves of every chunk (kh); b's fragments come from
// ds_read_b64_tr_b8 (eight consecutive reduction steps of one column per lane), a's from ds_read_b128.
#pragma once
#include "common.h"
#include "lds_asm.h"

namespace niti {

constexpr int kLinesStage = 128 * 128 + 32 * 128;   // bytes: b chunk, then a chunk
constexpr int kLinesRing = 3;
constexpr int kLinesLdsBytes = kLinesRing * kLinesStage;

__device__ inline void lines_sync() {   // barrier that the compiler also treats as a fence for the hand-written LDS reads
  asm volatile("" ::: "memory");
  __syncthreads();
  asm volatile("" ::: "memory");
}

// Returns every wavefront's partial product over its half of the chunks' steps (lines_add_halves adds the two).
// Element 4 q + e of a lane is column n0 + 32 ft + 8 q + 4 (lane / 32) + e of row m0 + lane % 32, with
// ft = wavefront % 4 and kh = wavefront / 4.  chunk0 / nchunks: the range of 128-step chunks.  Rows of a beyond m read
// as zeros.  m k and k n must be below 2^31 (buffer offsets).  smem: kLinesLdsBytes, 16-byte aligned; on return every
// wavefront has passed a barrier behind its last read of it.
__device__ inline v16i lines_product(const int8_t* a, const int8_t* b, int m, int n, int k, int m0, int n0, int chunk0, int nchunks,
                                     int8_t* smem) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(b), 0, k * n, 0x00020000);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a), 0, m * k, 0x00020000);
  // staging: 20 instructions per chunk (16 of b's rows, 4 of a's rows), wavefront w issues numbers w, w + 8, w + 16
  const int r8 = lane >> 3, piece = (lane & 7) ^ r8;
  constexpr int kFar = static_cast<int>(0x80000000u);   // out of range whatever scalar offset is added: zeros
  const int src0 = (8 * wave + r8) * n + n0 + piece * 16;
  const int src1 = (8 * (wave + 8) + r8) * n + n0 + piece * 16;
  // a's rows: swizzled by row / 2, since their readers take 16 bytes of 16 consecutive rows at once
  const int apiece = (lane & 7) ^ ((4 * (wave & 1) + (r8 >> 1)) & 7);
  const int src2 = m0 + 8 * wave + r8 < m ? (m0 + 8 * wave + r8) * k + apiece * 16 : kFar;
  const unsigned lds0 = lds_addr(smem);
  auto issue = [&](int c, int st) {
    const unsigned dst = lds0 + st * kLinesStage;
    const int bo = (chunk0 + c) * 128 * n, ao = (chunk0 + c) * 128;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, NITI_LDS_AT(dst + wave * 1024), 16, src0, bo, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, NITI_LDS_AT(dst + (wave + 8) * 1024), 16, src1, bo, 0, 0);
    if (wave < 4) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, NITI_LDS_AT(dst + 16384 + wave * 1024), 16, src2, ao, 0, 0);
  };
  const int ft = wave & 3, kh = wave >> 2;
  const int lr = lane & 31, lk = lane >> 5;
  const int j = lane & 15, gg = (lane >> 4) & 1;
  // b chunk row kh * 64 + s * 32 + lk * 16 + (j >> 1) (+ 8), bytes ft * 32 + gg * 16 + 8 (j & 1) .. + 8
  const unsigned b_off = static_cast<unsigned>((kh * 64 + lk * 16 + (j >> 1)) * 128 + (((ft * 2 + gg) ^ (j >> 1)) << 4) + 8 * (j & 1));
  // a chunk row lr, bytes kh * 64 + s * 32 + lk * 16 .. + 16
  unsigned a_off[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) a_off[s] = static_cast<unsigned>(16384 + lr * 128 + (((kh * 4 + s * 2 + lk) ^ ((lr >> 1) & 7)) << 4));
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  issue(0, 0);
  if (nchunks > 1) issue(1, 1);
  for (int c = 0; c < nchunks; ++c) {
    // younger than this chunk's loads: the next chunk's (3 per wavefront 0 - 3, 2 per wavefront 4 - 7)
    if (c + 1 < nchunks) {
      if (wave < 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 3);
      else __builtin_amdgcn_s_waitcnt(0x0F70 | 2);
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    lines_sync();   // the chunk has landed for every wavefront, and the stage refilled below has been read by all
    if (c + 2 < nchunks) issue(c + 2, (c + 2) % kLinesRing);
    const unsigned base = lds0 + (c % kLinesRing) * kLinesStage;
    v2i lo[2], hi[2];
    v4i fa[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      lo[s] = lds_read_tr8<0>(base + b_off + s * 4096);
      hi[s] = lds_read_tr8<1024>(base + b_off + s * 4096);
      fa[s] = lds_read_b128(base + a_off[s]);
    }
    lds_settle<0>();
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      asm volatile("" : "+v"(fa[s]));
      // MFMA A = 32 columns of c x 32 reduction steps, B = 32 rows of c x 32 steps
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(lds_landed(lo[s], hi[s]), fa[s], acc, 0, 0, 0);
    }
  }
  lines_sync();   // every wavefront is done with the stages
  return acc;
}

// Adds the two halves of every chunk: on return the wavefronts with kh == 0 hold the sums; 16 KB at the start of smem
// are used, and a barrier follows the last read of them only when the caller places one.
__device__ inline void lines_add_halves(v16i& acc, int8_t* smem) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int* const park = reinterpret_cast<int*>(smem) + (wave & 3) * (16 * 64) + lane;
  if ((wave >> 2) == 1) {
#pragma unroll
    for (int e = 0; e < 16; ++e) park[e * 64] = acc[e];
  }
  __syncthreads();
  if ((wave >> 2) == 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] += park[e * 64];
  }
}

}  // namespace niti
