/*
 * CPU oracle for NITI's int8 hot path, plain C -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this
 * library.  It restates, as closed forms on machine integers, what the reference's
 * Python does with chains of torch elementwise ops, and what its CUDA extensions compute
 * through CUTLASS / cuBLAS / cuDNN.  It is written independently of oracle/niti_oracle.py
 * (which replays the literal torch op sequence); the tests check the two against each
 * other and against hand-derived known answers.
 *
 * Layouts: activations NHWC int8, filters KRSC int8, conv results NPQK int32.
 * div_mode: 0 = floor (torch >= 1.13 meaning of `//`), 1 = trunc (torch <= 1.12).
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   nito_round_shift   ti_torch.py:23-31        nito_sto_shift     ti_torch.py:33-46
 *   nito_psto_shift    ti_torch.py:48-69        nito_bitwidth_*    ti_torch.py:366-377
 *   nito_requant       ti_torch.py:103-147      nito_weight_update ti_torch.py:21
 *   nito_conv_fprop    pytorch/cutlass-extension/cutlassconv_kernel.cu:107-148
 *   nito_conv_dgrad    ti_torch.py:403-405 (as the true data gradient, any stride)
 *   nito_conv_wgrad    ti_torch.py:430-432 / 194-233 (as the true weight gradient)
 *   nito_f32_roundtrip include/cutlass/epilogue/thread/linear_combination_clamp.h:371-389
 *   nito_gemm          pytorch/int8mm-extension/int8mm_kernel.cu:8-34
 *   nito_maxpool_*     pytorch/int8pool-extension/int8pool_kernel.cu:28-138
 *                      (backward tie rule: parity unpinned, see niti_oracle.py header)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int nito_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------- scalar helpers */
static inline int8_t clip127(int64_t v) { return (int8_t)(v > 127 ? 127 : (v < -127 ? -127 : v)); }
static inline int64_t sgn64(int64_t v) { return (v > 0) - (v < 0); }

/* quotient and non-negative remainder magnitude of x / 2^s under the two division modes */
static inline void split_pow2(int64_t x, int s, int trunc, int64_t* q, int64_t* rem_abs) {
  if (!trunc || x >= 0) {
    *q = x >> s;                       /* arithmetic shift == floor */
    *rem_abs = x - (*q << s);          /* in [0, 2^s) */
  } else {
    int64_t a = -x;
    *q = -(a >> s);
    *rem_abs = a & (((int64_t)1 << s) - 1);
  }
}

int8_t nito_round_shift1(int32_t x, int s, int trunc) {
  int64_t half = (int64_t)1 << (s - 1);
  if (!trunc) return clip127(((int64_t)x + half) >> s);                 /* round half up */
  int64_t a = x < 0 ? -(int64_t)x : (int64_t)x;                         /* round half away */
  return clip127(sgn64(x) * ((a + half) >> s));
}

int8_t nito_sto_shift1(int32_t x, int s, int32_t u, int trunc) {
  int64_t q, rem;
  split_pow2(x, s, trunc, &q, &rem);
  return clip127(q + (rem > (int64_t)u ? sgn64(x) : 0));
}

int8_t nito_psto_shift1(int32_t x, int s, int trunc) {
  int64_t q, rem;
  split_pow2(x, s, trunc, &q, &rem);
  int h = s / 2;
  int64_t hi = rem >> h;
  int64_t lo = rem & (((int64_t)1 << h) - 1);
  if (s & 1) lo <<= 1;
  return clip127(q + (hi > lo ? sgn64(x) : 0));
}

void nito_round_shift(const int32_t* x, int8_t* y, int64_t n, int s, int trunc) {
  for (int64_t i = 0; i < n; ++i) y[i] = nito_round_shift1(x[i], s, trunc);
}
void nito_sto_shift(const int32_t* x, const int32_t* u, int8_t* y, int64_t n, int s, int trunc) {
  for (int64_t i = 0; i < n; ++i) y[i] = nito_sto_shift1(x[i], s, u[i], trunc);
}
void nito_psto_shift(const int32_t* x, int8_t* y, int64_t n, int s, int trunc) {
  for (int64_t i = 0; i < n; ++i) y[i] = nito_psto_shift1(x[i], s, trunc);
}

/* ceil(log2(r)) for r >= 1 as an exact integer; 0 for r == 0 */
int nito_bitwidth_int(uint32_t r) {
  if (r <= 1) return 0;
  int b = 0;
  uint32_t v = r - 1;
  while (v) { ++b; v >>= 1; }
  return b;
}

/* the reference's literal evaluation int(ceil(log2f((float)r))) with this libm */
int nito_bitwidth_f32_libm(uint32_t r) {
  if (r == 0) return 0;
  return (int)ceilf(log2f((float)r));
}

uint32_t nito_absmax(const int32_t* x, int64_t n) {
  uint32_t m = 0;
  for (int64_t i = 0; i < n; ++i) {
    uint32_t a = x[i] < 0 ? (uint32_t)(-(int64_t)x[i]) : (uint32_t)x[i];
    if (a > m) m = a;
  }
  return m;
}

/*
 * act_calc / err_calc / grad_calc in one routine: shift = bitwidth(max|x|) - target_bits.
 * shift >= 1: apply the rounding method (0 round, 1 sto, 2 psto); otherwise keep the low
 * byte (the reference's `.type(torch.int8)`, 128 wraps to -128).  Returns max(shift, 0).
 */
int nito_requant(const int32_t* x, const int32_t* u, int8_t* y, int64_t n, int target_bits, int method,
                 int trunc) {
  int shift = nito_bitwidth_int(nito_absmax(x, n)) - target_bits;
  if (shift < 1) {
    for (int64_t i = 0; i < n; ++i) y[i] = (int8_t)(uint8_t)(x[i] & 0xFF);
    return 0;
  }
  if (method == 0) nito_round_shift(x, y, n, shift, trunc);
  else if (method == 1) nito_sto_shift(x, u, y, n, shift, trunc);
  else nito_psto_shift(x, y, n, shift, trunc);
  return shift;
}

void nito_weight_update(int8_t* w, const int8_t* g, int64_t n) {
  for (int64_t i = 0; i < n; ++i) w[i] = clip127((int64_t)w[i] - (int64_t)g[i]);
}

/* int32 -> fp32 (RNE) -> clamp -> nearest int32, saturating */
void nito_f32_roundtrip(const int32_t* x, int32_t* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float f = (float)x[i];
    if (f >= 2147483648.0f) y[i] = INT32_MAX;
    else if (f <= -2147483648.0f) y[i] = INT32_MIN;
    else y[i] = (int32_t)lrintf(f);
  }
}

/* ---------------------------------------------------------------- convolution */
static inline int out_dim(int in, int pad, int k, int stride) { return (in + 2 * pad - k) / stride + 1; }

/* y[n,p,q,k] = sum_{r,s,c} x[n, p*st-pad+r, q*st-pad+s, c] * w[k,r,s,c] */
void nito_conv_fprop(const int8_t* x, const int8_t* w, int32_t* y, int N, int H, int W, int C, int K, int R,
                     int S, int stride, int pad) {
  const int P = out_dim(H, pad, R, stride), Q = out_dim(W, pad, S, stride);
  /* re-lay the filter as [r][s][c][k] int16 so the innermost loop runs over k */
  int16_t* wt = (int16_t*)malloc(sizeof(int16_t) * (size_t)R * S * C * K);
  for (int k = 0; k < K; ++k)
    for (int r = 0; r < R; ++r)
      for (int s = 0; s < S; ++s)
        for (int c = 0; c < C; ++c)
          wt[(((size_t)r * S + s) * C + c) * K + k] = w[(((size_t)k * R + r) * S + s) * C + c];
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n)
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q) {
        int32_t* acc = y + (((size_t)n * P + p) * Q + q) * K;
        memset(acc, 0, sizeof(int32_t) * K);
        for (int r = 0; r < R; ++r) {
          int h = p * stride - pad + r;
          if (h < 0 || h >= H) continue;
          for (int s = 0; s < S; ++s) {
            int ww = q * stride - pad + s;
            if (ww < 0 || ww >= W) continue;
            const int8_t* xp = x + (((size_t)n * H + h) * W + ww) * C;
            const int16_t* wp = wt + ((size_t)r * S + s) * C * K;
            for (int c = 0; c < C; ++c) {
              const int32_t xv = xp[c];
              const int16_t* wk = wp + (size_t)c * K;
              for (int k = 0; k < K; ++k) acc[k] += xv * wk[k];
            }
          }
        }
      }
  free(wt);
}

/* dx[n,h,w,c] = sum over (p,q,r,s,k) with h = p*st-pad+r, w = q*st-pad+s of err[n,p,q,k] * w[k,r,s,c] */
void nito_conv_dgrad(const int8_t* err, const int8_t* w, int32_t* dx, int N, int H, int W, int C, int K,
                     int R, int S, int stride, int pad) {
  const int P = out_dim(H, pad, R, stride), Q = out_dim(W, pad, S, stride);
  int16_t* w16 = (int16_t*)malloc(sizeof(int16_t) * (size_t)K * R * S * C);
  for (size_t i = 0; i < (size_t)K * R * S * C; ++i) w16[i] = w[i];
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n)
    for (int h = 0; h < H; ++h)
      for (int ww = 0; ww < W; ++ww) {
        int32_t* acc = dx + (((size_t)n * H + h) * W + ww) * C;
        memset(acc, 0, sizeof(int32_t) * C);
        for (int r = 0; r < R; ++r) {
          int ph = h + pad - r;
          if (ph < 0 || ph % stride) continue;
          int p = ph / stride;
          if (p >= P) continue;
          for (int s = 0; s < S; ++s) {
            int qw = ww + pad - s;
            if (qw < 0 || qw % stride) continue;
            int q = qw / stride;
            if (q >= Q) continue;
            const int8_t* ep = err + (((size_t)n * P + p) * Q + q) * K;
            for (int k = 0; k < K; ++k) {
              const int32_t ev = ep[k];
              const int16_t* wc = w16 + (((size_t)k * R + r) * S + s) * C;
              for (int c = 0; c < C; ++c) acc[c] += ev * wc[c];
            }
          }
        }
      }
  free(w16);
}

/* dw[k,r,s,c] = sum_{n,p,q} err[n,p,q,k] * act[n, p*st-pad+r, q*st-pad+s, c] */
void nito_conv_wgrad(const int8_t* act, const int8_t* err, int32_t* dw, int N, int H, int W, int C, int K,
                     int R, int S, int stride, int pad) {
  const int P = out_dim(H, pad, R, stride), Q = out_dim(W, pad, S, stride);
  memset(dw, 0, sizeof(int32_t) * (size_t)K * R * S * C);
#pragma omp parallel for schedule(dynamic, 1)
  for (int k0 = 0; k0 < K; k0 += 4) {
    const int kn = K - k0 < 4 ? K - k0 : 4;
    for (int n = 0; n < N; ++n)
      for (int p = 0; p < P; ++p)
        for (int q = 0; q < Q; ++q) {
          const int8_t* ep = err + (((size_t)n * P + p) * Q + q) * K + k0;
          for (int r = 0; r < R; ++r) {
            int h = p * stride - pad + r;
            if (h < 0 || h >= H) continue;
            for (int s = 0; s < S; ++s) {
              int ww = q * stride - pad + s;
              if (ww < 0 || ww >= W) continue;
              const int8_t* ap = act + (((size_t)n * H + h) * W + ww) * C;
              for (int kk = 0; kk < kn; ++kk) {
                const int32_t ev = ep[kk];
                if (!ev) continue;
                int32_t* d = dw + ((((size_t)(k0 + kk)) * R + r) * S + s) * C;
                for (int c = 0; c < C; ++c) d[c] += ev * ap[c];
              }
            }
          }
        }
  }
}

/* c[m,n] = sum_k a[m,k] * b[k,n], row-major, exact int32 */
void nito_gemm(const int8_t* a, const int8_t* b, int32_t* c, int m, int n, int k) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < m; ++i) {
    int32_t* ci = c + (size_t)i * n;
    memset(ci, 0, sizeof(int32_t) * n);
    for (int kk = 0; kk < k; ++kk) {
      const int32_t av = a[(size_t)i * k + kk];
      const int8_t* bk = b + (size_t)kk * n;
      for (int j = 0; j < n; ++j) ci[j] += av * bk[j];
    }
  }
}

/* ---------------------------------------------------------------- max-pool (NHWC int8) */
void nito_maxpool_fwd(const int8_t* x, int8_t* y, int N, int H, int W, int C, int ks, int stride, int pad) {
  const int P = out_dim(H, pad, ks, stride), Q = out_dim(W, pad, ks, stride);
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n)
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q)
        for (int c = 0; c < C; ++c) {
          int best = -129;
          for (int kh = 0; kh < ks; ++kh) {
            int h = p * stride - pad + kh;
            if (h < 0 || h >= H) continue;
            for (int kw = 0; kw < ks; ++kw) {
              int w = q * stride - pad + kw;
              if (w < 0 || w >= W) continue;
              int v = x[(((size_t)n * H + h) * W + w) * C + c];
              if (v > best) best = v;
            }
          }
          y[(((size_t)n * P + p) * Q + q) * C + c] = (int8_t)best;
        }
}

/* ties_all == 0: first maximum in (kh,kw) scan order receives dy; 1: every maximum does */
void nito_maxpool_bwd(const int8_t* y, const int8_t* dy, const int8_t* x, int8_t* dx, int N, int H, int W,
                      int C, int ks, int stride, int pad, int ties_all) {
  const int P = out_dim(H, pad, ks, stride), Q = out_dim(W, pad, ks, stride);
  int32_t* acc = (int32_t*)calloc((size_t)N * H * W * C, sizeof(int32_t));
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n)
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q)
        for (int c = 0; c < C; ++c) {
          size_t o = (((size_t)n * P + p) * Q + q) * C + c;
          int done = 0;
          for (int kh = 0; kh < ks && !(done && !ties_all); ++kh) {
            int h = p * stride - pad + kh;
            if (h < 0 || h >= H) continue;
            for (int kw = 0; kw < ks; ++kw) {
              int w = q * stride - pad + kw;
              if (w < 0 || w >= W) continue;
              size_t i = (((size_t)n * H + h) * W + w) * C + c;
              if (x[i] == y[o] && (ties_all || !done)) {
                acc[i] += dy[o];
                done = 1;
              }
            }
          }
        }
  for (size_t i = 0; i < (size_t)N * H * W * C; ++i) dx[i] = (int8_t)acc[i];
  free(acc);
}

/* ---------------------------------------------------------------- integer cross-entropy gradient (ti_loss.py:5-36) */
/* 2^s of ti_loss.py:24 as a fixed sequence of IEEE double operations (built with -ffp-contract=off): n = floor(s),
 * x = (s - n) ln2, Horner's rule over 1/k! (k = 18 .. 0) with one rounded product and one rounded sum per step,
 * result = (float)(p 2^n).  The HIP kernel runs the same sequence, so host and device agree bit for bit. */
static const double k_exp2_coef[19] = {
    0x1.0000000000000p+0,  0x1.0000000000000p+0,  0x1.0000000000000p-1,  0x1.5555555555555p-3,  0x1.5555555555555p-5,
    0x1.1111111111111p-7,  0x1.6c16c16c16c17p-10, 0x1.a01a01a01a01ap-13, 0x1.a01a01a01a01ap-16, 0x1.71de3a556c734p-19,
    0x1.27e4fb7789f5cp-22, 0x1.ae64567f544e4p-26, 0x1.1eed8eff8d898p-29, 0x1.6124613a86d09p-33, 0x1.93974a8c07c9dp-37,
    0x1.ae7f3e733b81fp-41, 0x1.ae7f3e733b81fp-45, 0x1.952c77030ad4ap-49, 0x1.6827863b97d97p-53};

float nito_exp2_contract(float s) {
  const double d = (double)s;
  const double n = floor(d);
  const double x = (d - n) * 0x1.62e42fefa39efp-1;
  volatile double p = k_exp2_coef[18];
  for (int k = 17; k >= 0; --k) {
    p = p * x;
    p = p + k_exp2_coef[k];
  }
  return (float)ldexp(p, (int)n);
}

/* everything before the final StoShift: pre[n][classes] is the int32 tensor of ti_loss.py:35.  Every float
 * operation is one float32 operation of the reference's tensor sequence, in its order. */
void nito_ti_loss_pre_round(const int8_t* out, int n, int classes, int out_exp, const int64_t* target, int32_t* pre) {
  for (int i = 0; i < n; ++i) {
    const int8_t* v = out + (size_t)i * classes;
    int32_t* o = pre + (size_t)i * classes;
    volatile float num[1024];   /* numerators as float32 (volatile: no excess precision, no contraction) */
    int64_t out_sum = 0;
    if (classes > 1024) return;
    if (out_exp > -7) {
      const float p2 = ldexpf(1.0f, out_exp >= 0 ? out_exp : -out_exp);
      float mx = -INFINITY;
      for (int j = 0; j < classes; ++j) {
        volatile float s = (float)((int64_t)v[j] * 47274) / 32768.0f;     /* :14 */
        s = out_exp >= 0 ? s * p2 : s / p2;                               /* :15-18 */
        num[j] = s;
        if (s > mx) mx = s;
      }
      volatile float offset = mx - 10.0f;                                  /* :20-21 */
      for (int j = 0; j < classes; ++j) {
        volatile float s = num[j] - offset;                                /* :22 */
        if (s < 0.0f) s = 0.0f;                                            /* :23 */
        volatile float pw = nito_exp2_contract(s);
        num[j] = pw - 1.0f;                                                /* :24 */
        out_sum += (int64_t)num[j];                                        /* :31 */
      }
    } else {
      for (int j = 0; j < classes; ++j) {
        const int64_t x = v[j];
        const int64_t t = ((int64_t)1 << (1 - 2 * out_exp)) + x * ((int64_t)1 << (1 - out_exp)) + x * x;   /* :28-29 */
        out_sum += t;
        num[j] = (float)t;   /* :33 multiplies in int64 first; float(2048 t) = 2048 float(t), a power of two */
      }
    }
    const float fsum = (float)out_sum;
    int64_t tsum = 0;
    for (int j = 0; j < classes; ++j) {
      volatile float prod = num[j] * 2048.0f;
      num[j] = prod / fsum;                                                /* :33 */
      tsum += (int64_t)num[j];                                             /* :34 */
    }
    for (int j = 0; j < classes; ++j) {
      volatile float g = num[j];
      if (j == target[i]) g = g - (float)tsum;                             /* :34 */
      o[j] = (int32_t)g;                                                   /* :35 */
    }
  }
}

/* ---------------------------------------------------------------- float -> int8 quantisers */
/* ceil(log2 r) of a positive float from its exponent and mantissa (the exact value of ti_torch.py:336,348) */
int nito_ceil_log2_f32(float r) {
  int e;
  const float m = frexpf(r, &e);   /* r = m 2^e, 0.5 <= m < 1 */
  return m == 0.5f ? e - 1 : e;
}

/* TiFloatToInt8 (ti_torch.py:341-356) on a flat array; returns the exponent bw - bits (0 for an all-zero input) */
int nito_float_to_int8(const float* x, int8_t* y, int64_t n, int bits) {
  float r = 0.0f;
  for (int64_t i = 0; i < n; ++i) r = fabsf(x[i]) > r ? fabsf(x[i]) : r;
  if (r == 0.0f) {
    memset(y, 0, (size_t)n);
    return 0;
  }
  const int bw = nito_ceil_log2_f32(r);
  const float scale = ldexpf(1.0f, bits - bw);
  for (int64_t i = 0; i < n; ++i) {
    float q = nearbyintf(x[i] * scale);   /* round half to even in the default rounding mode */
    q = q < -128.0f ? -128.0f : (q > 127.0f ? 127.0f : q);
    y[i] = (int8_t)q;
  }
  return bw - bits;
}

/* weight_quant (ti_torch.py:334-339); returns the exponent */
int nito_weight_quant(const float* w, int8_t* y, int64_t n) {
  float r = 0.0f;
  for (int64_t i = 0; i < n; ++i) r = fabsf(w[i]) > r ? fabsf(w[i]) : r;
  for (int64_t i = 0; i < n; ++i) {
    volatile float q = w[i] / r;
    q = q * 127.0f;
    y[i] = (int8_t)nearbyintf(q);
  }
  return nito_ceil_log2_f32(r) - 7;
}
