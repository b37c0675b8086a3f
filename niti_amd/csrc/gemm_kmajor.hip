// int8 GEMM with int32 results for operands whose reduction index is the slow one, read as they are stored:
//   NN  c[m][n] = sum_k a[m][k] b[k][n]   - the form the reference's extension receives (int8mm.cpp:9-14,
//       int8mm_kernel.cu:8-34; ti_torch.py:152-176 hands it row-major [m,k] and [k,n])
//   TN  c[m][n] = sum_k a[k][m] b[k][n]
//   TT  c[m][n] = sum_k a[k][m] b[n][k]   - the NN product of (b, a) written transposed: how the drop-in int8_mm
//       fills the [n,m] buffer whose transposed view the reference returns (int8mm.cpp:9-14)
// A workgroup owns MT x 32 rows x 32 columns of c.  It stages b[k0 .. k0+chunk)[n0 .. n0+32) as stored - rows of 32
// bytes - and builds the MFMA fragments with ds_read_b64_tr_b8, which hands each lane eight consecutive rows of one
// byte column; in the TN form the workgroup's columns of a are staged the same way (rows padded by 16 bytes: eight
// consecutive rows fall into eight different bank groups), in the NN form a's rows are reduction-contiguous and come
// straight from memory.  8 wavefronts = MT tiles of 32 rows x 8 / MT parts of each chunk's reduction steps, added
// through LDS at the end: MT = 4 in general, MT = 1 for a small result with a long reduction (the forward product of
// a fully connected layer on a batch), which would otherwise occupy a few workgroups.
// No operand is copied into another layout and the output is written once.
#include "common.h"
#include "lds_asm.h"
#include "nn_lines.h"

namespace niti {
namespace {

constexpr int kKmChunkNN = 2048;             // reduction rows staged at a time: 64 KB of b
constexpr int kKmChunkTN = 512;              // 16 KB of b + up to 72 KB of a

struct KmArgs {
  const int8_t* a;
  const int8_t* b;
  int32_t* c;
  uint32_t* absmax;
  int m, n, k;
  int roundtrip;
  int transposed_out;   // element (row, column) goes to c[column * m + row]
};

__device__ inline void km_sync() {
  asm volatile("" ::: "memory");
  __syncthreads();
  asm volatile("" ::: "memory");
}

template <bool kTransA, int MT>
__global__ __launch_bounds__(512) void gemm_kmajor_kernel(const KmArgs g) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  constexpr int CHUNK = kTransA ? kKmChunkTN : kKmChunkNN;
  constexpr int KS = 8 / MT;                   // parts of the reduction
  constexpr int kKmPitchA = MT * 32 + 16;
  int8_t* const a_s = smem + CHUNK * 32;     // TN only
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * 32;
  const int mb = blockIdx.y * (MT * 32);
  const int mt = wave % MT, kh = wave / MT;
  const int lr = lane & 31, lk = lane >> 5;
  const int j = lane & 15, gg = (lane >> 4) & 1;
  const int m = mb + mt * 32 + lr;
  const bool vm = m < g.m;
  const int8_t* const pa = g.a + static_cast<long long>(vm ? m : 0) * g.k + lk * 16;   // NN only
  const unsigned bbase = lds_addr(smem) + (lk * 16 + (j >> 1)) * 32 + gg * 16 + 8 * (j & 1);
  const unsigned abase = lds_addr(a_s) + (lk * 16 + (j >> 1)) * kKmPitchA + mt * 32 + gg * 16 + 8 * (j & 1);
  const v4i zero = {0, 0, 0, 0};
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;

  // a chunk travels memory -> registers -> LDS; the next chunk's loads are in flight while this one multiplies
  constexpr int NPB = CHUNK * 2 / 512;                 // 16-byte pieces of b per thread and chunk
  constexpr int NPA = kTransA ? CHUNK * 2 * MT / 512 : 1;
  v4i pre_b[NPB], pre_a[NPA];
  auto fetch = [&](int k0) {
    const int rows = min(CHUNK, g.k - k0);
#pragma unroll
    for (int i = 0; i < NPB; ++i) {
      const int p = tid + i * 512;
      const int r = p >> 1, half = p & 1;
      pre_b[i] = r < rows ? *reinterpret_cast<const v4i*>(g.b + static_cast<long long>(k0 + r) * g.n + n0 + half * 16) : zero;
    }
    if (kTransA) {
#pragma unroll
      for (int i = 0; i < NPA; ++i) {
        const int p = tid + i * 512;
        const int r = p / (2 * MT), piece = p % (2 * MT);
        const int col = mb + piece * 16;               // m is a multiple of 16: a piece is inside or outside
        pre_a[i] = (r < rows && col < g.m) ? *reinterpret_cast<const v4i*>(g.a + static_cast<long long>(k0 + r) * g.m + col) : zero;
      }
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < g.k; k0 += CHUNK) {
    const int rows = min(CHUNK, g.k - k0);             // a multiple of 32
    if (k0 > 0) km_sync();                             // every wavefront is done with the previous chunk
#pragma unroll
    for (int i = 0; i < NPB; ++i) {
      const int p = tid + i * 512;
      *reinterpret_cast<v4i*>(smem + (p >> 1) * 32 + (p & 1) * 16) = pre_b[i];
    }
    if (kTransA) {
#pragma unroll
      for (int i = 0; i < NPA; ++i) {
        const int p = tid + i * 512;
        *reinterpret_cast<v4i*>(a_s + (p / (2 * MT)) * kKmPitchA + (p % (2 * MT)) * 16) = pre_a[i];
      }
    }
    km_sync();
    if (k0 + CHUNK < g.k) fetch(k0 + CHUNK);
    const int nsteps = rows >> 5;
    const int per = (nsteps + KS - 1) / KS;
    const int s0 = min(kh * per, nsteps);
    const int s1 = min(s0 + per, nsteps);
    for (int sb = s0; sb < s1; sb += 4) {              // four steps at a time, their loads in flight together
      v4i fa[4];
      v2i blo[4], bhi[4], alo[4], ahi[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = min(sb + u, nsteps - 1);
        blo[u] = lds_read_tr8<0>(bbase + static_cast<unsigned>(s) * 1024u);
        bhi[u] = lds_read_tr8<256>(bbase + static_cast<unsigned>(s) * 1024u);
        if (kTransA) {
          alo[u] = lds_read_tr8<0>(abase + static_cast<unsigned>(s) * (32u * kKmPitchA));
          ahi[u] = lds_read_tr8<8 * kKmPitchA>(abase + static_cast<unsigned>(s) * (32u * kKmPitchA));
        } else {
          fa[u] = (vm && sb + u < s1) ? *reinterpret_cast<const v4i*>(pa + k0 + (sb + u) * 32) : zero;
        }
      }
      lds_settle<0>();
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const v4i fb = lds_landed(blo[u], bhi[u]);
        if (kTransA) fa[u] = lds_landed(alo[u], ahi[u]);
        // MFMA A = 32 columns of c x 32 reduction steps, B = 32 rows of c x 32 steps
        if (sb + u < s1) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb, fa[u], acc, 0, 0, 0);
      }
    }
  }
  km_sync();   // every wavefront is done with the staged operands
  int* const park = reinterpret_cast<int*>(smem) + mt * (16 * 64) + lane;   // part p > 0 at park + (p - 1) * MT * 1024
  if (kh != 0) {
#pragma unroll
    for (int e = 0; e < 16; ++e) park[(kh - 1) * (MT * 1024) + e * 64] = acc[e];
  }
  __syncthreads();
  if (kh != 0) return;
  // element 4 q + e of a lane is column n0 + 8 q + 4 (lane / 32) + e of row m
  uint32_t lmax = 0;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    int v = acc[e];
#pragma unroll
    for (int p = 0; p < KS - 1; ++p) v += park[p * (MT * 1024) + e * 64];
    if (g.roundtrip) v = f32_roundtrip(v);
    acc[e] = v;
    const uint32_t u = uabs(v);                         // rows beyond m are sums of zeros
    lmax = u > lmax ? u : lmax;
  }
  if (g.absmax != nullptr) fold_absmax(g.absmax, lmax);
  if (!vm) return;
  if (g.transposed_out) {   // 32 lanes write 32 consecutive rows of one column
#pragma unroll
    for (int e = 0; e < 16; ++e)
      g.c[static_cast<long long>(n0 + 8 * (e >> 2) + 4 * lk + (e & 3)) * g.m + m] = acc[e];
    return;
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
    *reinterpret_cast<v4i*>(g.c + static_cast<long long>(m) * g.n + n0 + 8 * q + 4 * lk) =
        v4i{acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
}

// ---- NN form, both operands through LDS as whole 128-byte lines ------------------------------------------------------
// The kernel above stages b in 32-byte pieces of its rows and takes a in 32-byte pieces as well; the path from L2 into
// a compute unit moves such pieces at a quarter of the rate of whole lines.  Here (n and k multiples of 128) a workgroup
// owns 32 rows x 128 columns of c and a range of the reduction, and runs the whole-line product of nn_lines.h over it.
// blockIdx.z splits the reduction when the tiles alone would leave most of the device idle: the parts then write int32
// partial results and km_reduce_parts_kernel adds them.
constexpr int kLnPatchPitch = 128 * 4 + 16;

struct LnArgs {
  const int8_t* a;
  const int8_t* b;
  int32_t* out;           // c, or the partial results [part][m * n]
  uint32_t* absmax;
  int m, n, k;
  int chunks_per_part;
  int parts;
  int roundtrip;
  int transposed_out;
};

__global__ __launch_bounds__(512) void gemm_nn_lines_kernel(const LnArgs g) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];   // the stages; later 16 KB of parked sums, then the patch
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * 128;
  const int m0 = blockIdx.y * 32;
  const int c0 = blockIdx.z * g.chunks_per_part;
  const int nchunks = min(g.chunks_per_part, (g.k >> 7) - c0);
  const int ft = wave & 3, kh = wave >> 2;
  const int lr = lane & 31, lk = lane >> 5;
  v16i acc = lines_product(g.a, g.b, g.m, g.n, g.k, m0, n0, c0, nchunks, smem);
  lines_add_halves(acc, smem);
  // element 4 q + e of a lane is column n0 + ft * 32 + 8 q + 4 (lane / 32) + e of row m0 + lane % 32
  const bool last = g.parts == 1;
  int32_t* const out = g.out + static_cast<long long>(blockIdx.z) * g.m * g.n;
  int8_t* const patch = smem + 16384;                            // [32 rows][128 columns] of int32, clear of the parked sums
  if (kh == 0) {
    uint32_t lmax = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      int v = acc[e];
      if (last && g.roundtrip) v = f32_roundtrip(v);
      acc[e] = v;
      const uint32_t u = uabs(v);                         // rows beyond m are sums of zeros
      lmax = u > lmax ? u : lmax;
    }
    if (last && g.absmax != nullptr) fold_absmax(g.absmax, lmax);
    if (g.transposed_out) {   // 32 lanes write 32 consecutive rows of one column: a line
      if (m0 + lr < g.m) {
#pragma unroll
        for (int e = 0; e < 16; ++e)
          out[static_cast<long long>(n0 + ft * 32 + 8 * (e >> 2) + 4 * lk + (e & 3)) * g.m + m0 + lr] = acc[e];
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<v4i*>(patch + lr * kLnPatchPitch + (ft * 32 + 8 * q + 4 * lk) * 4) =
            v4i{acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
    }
  }
  if (g.transposed_out) return;
  __syncthreads();
  const int row = tid >> 4, p16 = tid & 15;
  if (m0 + row >= g.m) return;
#pragma unroll
  for (int i = 0; i < 2; ++i)
    *reinterpret_cast<v4i*>(out + static_cast<long long>(m0 + row) * g.n + n0 + (p16 + 16 * i) * 4) =
        *reinterpret_cast<const v4i*>(patch + row * kLnPatchPitch + (p16 + 16 * i) * 16);
}

// c[i] = sum over the parts of the partial results: two elements per thread (the result is small - many short
// wavefronts cover the device better than few long ones), the loads of eight parts in flight together
__global__ __launch_bounds__(256) void km_reduce_parts_kernel(const int32_t* __restrict__ part, int32_t* __restrict__ c, long long pairs, int parts,
                                                              int roundtrip, uint32_t* absmax) {
  const long long i = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  uint32_t lmax = 0;
  if (i < pairs) {
    v2i s = {0, 0};
    for (int p0 = 0; p0 < parts; p0 += 8) {
      v2i v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = p0 + u < parts ? p0 + u : p0;          // a repeated part is not added below
        v[u] = *reinterpret_cast<const v2i*>(part + 2 * (static_cast<long long>(p) * pairs + i));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (p0 + u < parts) s += v[u];
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      if (roundtrip) s[e] = f32_roundtrip(s[e]);
      const uint32_t u = uabs(s[e]);
      lmax = u > lmax ? u : lmax;
    }
    *reinterpret_cast<v2i*>(c + 2 * i) = s;
  }
  if (absmax != nullptr) fold_absmax(absmax, lmax);
}

constexpr size_t km_lds(bool trans_a, int mt) {
  const size_t stage = trans_a ? static_cast<size_t>(kKmChunkTN) * 32 + static_cast<size_t>(kKmChunkTN) * (mt * 32 + 16)
                               : static_cast<size_t>(kKmChunkNN) * 32;
  const size_t park = static_cast<size_t>(8 / mt - 1) * mt * 4096;
  return stage > park ? stage : park;
}

template <bool kTransA, int MT>
int km_launch(const KmArgs& g, hipStream_t stream) {
  static bool attr_set[kDeviceSlots] = {};
  bool& done = attr_set[device_slot()];
  constexpr size_t lds = km_lds(kTransA, MT);
  if (!done) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_kmajor_kernel<kTransA, MT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(lds)) != hipSuccess)
      return fail(NITI_ERR_LAUNCH, "gemm: cannot reserve %zu bytes of LDS", lds);
    done = true;
  }
  const dim3 grid(g.n / 32, (g.m + MT * 32 - 1) / (MT * 32));
  hipLaunchKernelGGL((gemm_kmajor_kernel<kTransA, MT>), grid, dim3(512), lds, stream, g);
  return check_launch("gemm_kmajor");
}

// The whole-line kernel's plan for an NN product (after the TT form has been turned into one): 0 parts = not taken.
struct LnPlan {
  int parts, chunks_per_part;
};
LnPlan lines_plan(int m, int n, int k) {
  LnPlan p{0, 0};
  if (n % 128 != 0 || k % 128 != 0 || (m + 31) / 32 > 65535) return p;
  if (static_cast<long long>(m) * k >= 0x7fffffffLL || static_cast<long long>(k) * n >= 0x7fffffffLL) return p;
  static const bool off = [] {
    const char* e = getenv("NITI_GEMM_LINES");
    return e != nullptr && e[0] == '0';
  }();
  if (off) return p;
  const long long tiles = static_cast<long long>(n / 128) * ((m + 31) / 32);
  const int chunks = k / 128;
  int parts = 1;
  if (tiles < 192) {
    parts = static_cast<int>((256 + tiles - 1) / tiles);
    if (parts > chunks / 2) parts = chunks / 2;
    if (parts > 32) parts = 32;
    if (parts < 1) parts = 1;
  }
  p.chunks_per_part = (chunks + parts - 1) / parts;
  p.parts = (chunks + p.chunks_per_part - 1) / p.chunks_per_part;
  return p;
}

}  // namespace

// Shapes the direct kernels take: 32-column tiles, whole reduction steps, 16-byte pieces of every row.
bool gemm_kmajor_shape(int trans_a, int trans_b, int m, int n, int k) {
  if (m <= 0 || n <= 0 || k <= 0 || k % 32 != 0) return false;
  if (trans_b != 0) return trans_a != 0 && m % 32 == 0 && (n + 127) / 128 <= 65535;   // TT = NN of (b, a), transposed
  if (n % 32 != 0) return false;
  if (trans_a != 0 && m % 16 != 0) return false;
  return (m + 127) / 128 <= 65535;
}

// bytes of partial results the whole-line kernel wants for this product (0: none, or another kernel takes it)
size_t gemm_kmajor_workspace(int trans_a, int trans_b, int m, int n, int k) {
  if (trans_b != 0) {
    const int t = m;
    m = n;
    n = t;
    trans_a = 0;
  }
  if (trans_a != 0) return 0;
  const LnPlan p = lines_plan(m, n, k);
  return p.parts > 1 ? static_cast<size_t>(p.parts) * m * n * 4 : 0;
}

int launch_gemm_kmajor(int trans_a, int trans_b, const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k, bool roundtrip,
                       uint32_t* absmax, void* workspace, hipStream_t stream) {
  KmArgs g{a, b, c, absmax, m, n, k, roundtrip ? 1 : 0, 0};
  if (trans_b != 0) {   // rows of the kernel's product = n (rows of b), columns = m (columns of a)
    g.a = b;
    g.b = a;
    g.m = n;
    g.n = m;
    g.transposed_out = 1;
    trans_a = 0;
  }
  if (trans_a == 0) {
    const LnPlan p = lines_plan(g.m, g.n, k);
    if (p.parts > 0) {
      static bool attr_set[kDeviceSlots] = {};
      bool& done = attr_set[device_slot()];
      if (!done) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_nn_lines_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLinesLdsBytes) != hipSuccess)
          return fail(NITI_ERR_LAUNCH, "gemm: cannot reserve %d bytes of LDS", kLinesLdsBytes);
        done = true;
      }
      LnArgs l{g.a, g.b, p.parts > 1 ? static_cast<int32_t*>(workspace) : c, absmax, g.m, g.n, k, p.chunks_per_part, p.parts, g.roundtrip, g.transposed_out};
      hipLaunchKernelGGL(gemm_nn_lines_kernel, dim3(g.n / 128, (g.m + 31) / 32, p.parts), dim3(512), static_cast<size_t>(kLinesLdsBytes), stream, l);
      if (p.parts > 1) {
        const long long pairs = static_cast<long long>(g.m) * g.n / 2;
        hipLaunchKernelGGL(km_reduce_parts_kernel, dim3(static_cast<unsigned>((pairs + 255) / 256)), dim3(256), 0, stream,
                           static_cast<const int32_t*>(workspace), c, pairs, p.parts, g.roundtrip, absmax);
      }
      return check_launch("gemm_nn_lines");
    }
  }
  // few 128-row tiles and a long reduction: 32-row tiles whose eight wavefronts split the reduction
  const long long tiles128 = static_cast<long long>(g.n / 32) * ((g.m + 127) / 128);
  const bool thin = tiles128 < 128 && k >= 1024;
  if (trans_a != 0) return thin ? km_launch<true, 1>(g, stream) : km_launch<true, 4>(g, stream);
  return thin ? km_launch<false, 1>(g, stream) : km_launch<false, 4>(g, stream);
}

}  // namespace niti
