/*
 * kcg_oracle.c -- CPU restatement of the naive affine loop nests that the
 * KernelCodeGen Frontend emits (the functions it tags func.state = "cpu").
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the single-core CPU baseline that the benchmark times.
 * Nothing in the shipped library links, loads or calls it.
 *
 * Every routine follows the op-by-op order of the reference nest it cites and
 * is compiled with -ffp-contract=off so that a mulf followed by an addf stays
 * two IEEE roundings, exactly as arith.mulf / arith.addf lower without fusion.
 *
 * Pinning (how each routine is known to be right without running the
 * reference, whose own tests hold no numerical vector):
 *   matmul / batched matmul : brute-force tiny shapes, A*I = A, (AB)^T = B^T A^T,
 *                             linearity, agreement of the i-j-k nest with the
 *                             i-k-j interchange, fp64-accumulated truth.
 *   softmax                 : closed form on tiny rows, rows sum to 1,
 *                             shift invariance against a max-subtracted form.
 *   layernorm               : two hand-derived known answers, zero mean /
 *                             unit variance, invariance under a*x+b.
 *   gelu                    : eight known answers with the truncated constants.
 *   fmha                    : V constant => O constant, causal row 0 => V[0],
 *                             composition of the three nests above.
 *   bf16 / fp8 rounding     : exhaustive decode/encode round trip, ties-to-even
 *                             cases, saturation at 448.
 *   gather                  : numpy.take on the same operands (a library routine
 *                             of the same definition), identity indices, a
 *                             single index, a pure-Python loop on tiny shapes.
 * The checks live in tests/test_oracle.py.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KCG_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* Seeded synthetic inputs.                                                  */
/* splitmix64 counter stream: element i of stream s under seed z uses the    */
/* state z + (s << 40) + i, so any element can be generated independently.   */
/* uniform: top 24 bits / 2^24 in [0,1), then lo + (hi-lo)*u in fp32.        */
/* normal : Box-Muller in fp64 on two uniforms (53-bit), cast to fp32.       */
/* ------------------------------------------------------------------------ */
static inline uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

KCG_API void kcg_oracle_fill_uniform(float *dst, size_t n, uint64_t seed,
                                     uint64_t stream, float lo, float hi) {
  const uint64_t base = seed + (stream << 40);
  for (size_t i = 0; i < n; ++i) {
    uint64_t r = splitmix64(base + i);
    float u = (float)(r >> 40) * (1.0f / 16777216.0f);
    dst[i] = lo + (hi - lo) * u;
  }
}

KCG_API void kcg_oracle_fill_normal(float *dst, size_t n, uint64_t seed,
                                    uint64_t stream, float mean, float std) {
  const uint64_t base = seed + (stream << 40);
  const double two_pi = 6.283185307179586476925286766559;
  for (size_t i = 0; i < n; i += 2) {
    uint64_t r1 = splitmix64(base + i);
    uint64_t r2 = splitmix64(base + i + 1);
    double u1 = ((double)(r1 >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0,1] */
    double u2 = (double)(r2 >> 11) * (1.0 / 9007199254740992.0);         /* [0,1) */
    double rad = sqrt(-2.0 * log(u1));
    dst[i] = (float)((double)mean + (double)std * rad * cos(two_pi * u2));
    if (i + 1 < n)
      dst[i + 1] = (float)((double)mean + (double)std * rad * sin(two_pi * u2));
  }
}

/* ------------------------------------------------------------------------ */
/* Narrow float formats (additive dtypes; the reference knows only           */
/* float16/32/64, src/Frontend/Operators.cc:5-15).                           */
/* ------------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN. */
KCG_API uint16_t kcg_oracle_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu))
    return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7FFFu + lsb;
  return (uint16_t)(u >> 16);
}
KCG_API float kcg_oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

KCG_API void kcg_oracle_to_bf16(const float *src, uint16_t *dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = kcg_oracle_f32_to_bf16(src[i]);
}
KCG_API void kcg_oracle_from_bf16(const uint16_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = kcg_oracle_bf16_to_f32(src[i]);
}

/* OCP FP8 E4M3 "fn": bias 7, no infinities, 0x7F/0xFF are NaN, max 448. */
KCG_API float kcg_oracle_fp8e4m3_to_f32(uint8_t b) {
  uint32_t sign = (uint32_t)(b >> 7);
  uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
  float v;
  if (e == 0xF && m == 7) return u2f(0x7FC00000u | (sign << 31));
  if (e == 0) v = ldexpf((float)m, -9);               /* subnormal: m/8 * 2^-6 */
  else v = ldexpf(1.0f + (float)m * 0.125f, (int)e - 7);
  return sign ? -v : v;
}

/* fp32 -> e4m3fn, round to nearest even, saturating to +-448. */
KCG_API uint8_t kcg_oracle_f32_to_fp8e4m3(float f) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  float a = fabsf(f);
  if (a != a) return (uint8_t)(sign | 0x7Fu);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7Eu);
  if (a < ldexpf(1.0f, -10)) return sign;             /* below half the least subnormal */
  int ex;
  (void)frexpf(a, &ex);                               /* a = frac * 2^ex, frac in [0.5,1) */
  int e = ex - 1;                                     /* a = 1.x * 2^e */
  if (e < -6) e = -6;                                 /* subnormal grid */
  float q = ldexpf(a, 3 - e);                         /* units of 2^(e-3) */
  float r = nearbyintf(q);                            /* default mode: ties to even */
  int mant = (int)r;
  int be = e + 7;
  if (e == -6 && mant < 8) {                          /* subnormal result */
    return (uint8_t)(sign | (uint8_t)mant);
  }
  if (mant == 16) { mant = 8; be += 1; }
  if (be > 15 || (be == 15 && mant - 8 > 6)) return (uint8_t)(sign | 0x7Eu);
  return (uint8_t)(sign | (uint8_t)(be << 3) | (uint8_t)(mant - 8));
}
KCG_API void kcg_oracle_to_fp8e4m3(const float *src, uint8_t *dst, size_t n, float inv_scale) {
  for (size_t i = 0; i < n; ++i) dst[i] = kcg_oracle_f32_to_fp8e4m3(src[i] * inv_scale);
}
KCG_API void kcg_oracle_from_fp8e4m3(const uint8_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = kcg_oracle_fp8e4m3_to_f32(src[i]);
}

/* ------------------------------------------------------------------------ */
/* Matmul: C[i,j] = sum_k A[i,k]*B[k,j], accumulator starts at 0, k runs     */
/* sequentially, mulf then addf (src/Frontend/Operators.cc:186-210).         */
/* ------------------------------------------------------------------------ */

/* Literal nest order i, j, k: this is the loop nest the reference would      */
/* lower to the host; it is the routine the CPU baseline times.               */
KCG_API void kcg_oracle_matmul_f32_nest(const float *A, const float *B, float *C,
                                        int64_t M, int64_t N, int64_t K) {
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float mul = A[i * K + k] * B[k * N + j];
        acc = mul + acc;
      }
      C[i * N + j] = acc;
    }
}

/* Same arithmetic with the j and k loops interchanged.  Each C[i,j] still    */
/* adds its products in ascending k, so the result is bit-identical to the    */
/* nest above; only the memory walk differs.  The parity tests use this one.  */
KCG_API void kcg_oracle_matmul_f32(const float *A, const float *B, float *C,
                                   int64_t M, int64_t N, int64_t K) {
  for (int64_t i = 0; i < M; ++i) {
    float *c = C + i * N;
    for (int64_t j = 0; j < N; ++j) c[j] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const float a = A[i * K + k];
      const float *b = B + k * N;
      for (int64_t j = 0; j < N; ++j) {
        float mul = a * b[j];
        c[j] = mul + c[j];
      }
    }
  }
}

/* fp64-accumulated truth for the Frobenius metric (inputs are fp32 values). */
KCG_API void kcg_oracle_matmul_f64acc(const float *A, const float *B, double *C,
                                      int64_t M, int64_t N, int64_t K) {
  for (int64_t i = 0; i < M; ++i) {
    double *c = C + i * N;
    for (int64_t j = 0; j < N; ++j) c[j] = 0.0;
    for (int64_t k = 0; k < K; ++k) {
      const double a = (double)A[i * K + k];
      const float *b = B + k * N;
      for (int64_t j = 0; j < N; ++j) c[j] += a * (double)b[j];
    }
  }
}

/* Rows [row0, row0+rows) of C only: the bounded sample used at full sizes. */
KCG_API void kcg_oracle_matmul_rows_f64acc(const float *A, const float *B, double *Crows,
                                           int64_t row0, int64_t rows,
                                           int64_t N, int64_t K) {
  kcg_oracle_matmul_f64acc(A + row0 * K, B, Crows, rows, N, K);
}

/* ------------------------------------------------------------------------ */
/* BatchedMatmul (src/Frontend/Operators.cc:291-457): leading batch dims are  */
/* flattened to `batch`; transA / transB mirror Layout::colMajor.  For a      */
/* column-major A the element read is A[b, k, i]; the reference's nest reads  */
/* A[b, k, j] there (Operators.cc:427-429), which is out of bounds whenever   */
/* n > m and is not reproduced.                                               */
/* ------------------------------------------------------------------------ */
KCG_API void kcg_oracle_batched_matmul_f32(const float *A, const float *B, float *C,
                                           int64_t batch, int64_t M, int64_t N, int64_t K,
                                           int transA, int transB) {
  for (int64_t b = 0; b < batch; ++b) {
    const float *a_ = A + b * M * K;
    const float *b_ = B + b * K * N;
    float *c_ = C + b * M * N;
    for (int64_t i = 0; i < M; ++i)
      for (int64_t j = 0; j < N; ++j) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
          float av = transA ? a_[k * M + i] : a_[i * K + k];
          float bv = transB ? b_[j * K + k] : b_[k * N + j];
          float mul = av * bv;
          acc = mul + acc;
        }
        c_[i * N + j] = acc;
      }
  }
}

KCG_API void kcg_oracle_batched_matmul_f64acc(const float *A, const float *B, double *C,
                                              int64_t batch, int64_t M, int64_t N, int64_t K,
                                              int transA, int transB) {
  for (int64_t b = 0; b < batch; ++b) {
    const float *a_ = A + b * M * K;
    const float *b_ = B + b * K * N;
    double *c_ = C + b * M * N;
    for (int64_t i = 0; i < M; ++i)
      for (int64_t j = 0; j < N; ++j) {
        double acc = 0.0;
        for (int64_t k = 0; k < K; ++k) {
          double av = transA ? a_[k * M + i] : a_[i * K + k];
          double bv = transB ? b_[j * K + k] : b_[k * N + j];
          acc += av * bv;
        }
        c_[i * N + j] = acc;
      }
  }
}

/* ------------------------------------------------------------------------ */
/* Softmax over the last axis, in place (src/Frontend/Operators.cc:529-570):  */
/* sum = sum_k exp(x[k]) with NO max subtraction, then x[k] = exp(x[k])/sum.  */
/* ------------------------------------------------------------------------ */
KCG_API void kcg_oracle_softmax_f32(float *X, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    float *x = X + r * cols;
    float sum = 0.0f;
    for (int64_t k = 0; k < cols; ++k) sum = expf(x[k]) + sum;
    for (int64_t k = 0; k < cols; ++k) x[k] = expf(x[k]) / sum;
  }
}

KCG_API void kcg_oracle_softmax_f64(const float *X, double *Y, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *x = X + r * cols;
    double sum = 0.0;
    for (int64_t k = 0; k < cols; ++k) sum += exp((double)x[k]);
    for (int64_t k = 0; k < cols; ++k) Y[r * cols + k] = exp((double)x[k]) / sum;
  }
}

/* ------------------------------------------------------------------------ */
/* LayerNorm (src/Frontend/Operators.cc:1184-1241).  `rows` = product of the  */
/* dims before `axis`, `n` = product of the dims from `axis` on.              */
/*   pass 1: s = sum x (ascending), mean = s / n                              */
/*   pass 2: d = x - mean, STORED to y; v = sum d*d (mulf, addf), var = v / n */
/*   den = sqrt(var + eps)   (eps cast to the element type)                   */
/*   pass 3: y = gamma * (y / den) + beta   (divf, mulf, addf)                */
/* gamma/beta are broadcast over the trailing dims: element e of the          */
/* normalised group reads gamma[e % n_gamma] (n_gamma divides n when the      */
/* scale shape equals the trailing input dims).                               */
/* ------------------------------------------------------------------------ */
KCG_API void kcg_oracle_layernorm_f32(const float *X, const float *gamma, const float *beta,
                                      float *Y, int64_t rows, int64_t n,
                                      int64_t n_gamma, int64_t n_beta, float eps) {
  const float fn = (float)n;
  for (int64_t r = 0; r < rows; ++r) {
    const float *x = X + r * n;
    float *y = Y + r * n;
    float s = 0.0f;
    for (int64_t i = 0; i < n; ++i) s = x[i] + s;
    const float mean = s / fn;
    float v = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
      float d = x[i] - mean;
      y[i] = d;
      float sq = d * d;
      v = sq + v;
    }
    const float var = v / fn;
    const float den = sqrtf(var + eps);
    for (int64_t i = 0; i < n; ++i) {
      float q = y[i] / den;
      float m = gamma[i % n_gamma] * q;
      y[i] = m + beta[i % n_beta];
    }
  }
}

KCG_API void kcg_oracle_layernorm_f64(const float *X, const float *gamma, const float *beta,
                                      double *Y, int64_t rows, int64_t n,
                                      int64_t n_gamma, int64_t n_beta, double eps) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *x = X + r * n;
    double *y = Y + r * n;
    double s = 0.0;
    for (int64_t i = 0; i < n; ++i) s += (double)x[i];
    const double mean = s / (double)n;
    double v = 0.0;
    for (int64_t i = 0; i < n; ++i) { double d = (double)x[i] - mean; v += d * d; }
    const double den = sqrt(v / (double)n + eps);
    for (int64_t i = 0; i < n; ++i)
      y[i] = (double)gamma[i % n_gamma] * (((double)x[i] - mean) / den) + (double)beta[i % n_beta];
  }
}

/* ------------------------------------------------------------------------ */
/* ElementWise (src/Frontend/Operators.cc:960-1000) and Relu (:222-289).      */
/* GELU is the tanh form with the reference's truncated constants, in its op  */
/* order: t1 = x*0.5; t2 = x*x; t3 = x*t2; t4 = 0.044715*t3; t5 = t4+x;       */
/* t6 = 0.797884*t5; t7 = tanh(t6); t8 = t7+1; y = t1*t8.                     */
/* ------------------------------------------------------------------------ */
enum { KCG_EW_TANH = 0, KCG_EW_SQRT = 1, KCG_EW_LOG = 2, KCG_EW_RELU = 3, KCG_EW_GELU = 4 };

static inline float oracle_gelu(float x) {
  const float one = 1.0f, half = 0.5f, c0 = (float)0.797884, c1 = (float)0.044715;
  float t1 = x * half;
  float t2 = x * x;
  float t3 = x * t2;
  float t4 = c1 * t3;
  float t5 = t4 + x;
  float t6 = c0 * t5;
  float t7 = tanhf(t6);
  float t8 = t7 + one;
  return t1 * t8;
}

KCG_API float kcg_oracle_gelu_scalar(float x) { return oracle_gelu(x); }

KCG_API int kcg_oracle_elementwise_f32(const float *X, float *Y, size_t n, int op) {
  switch (op) {
    case KCG_EW_TANH: for (size_t i = 0; i < n; ++i) Y[i] = tanhf(X[i]); return 0;
    case KCG_EW_SQRT: for (size_t i = 0; i < n; ++i) Y[i] = sqrtf(X[i]); return 0;
    case KCG_EW_LOG:  for (size_t i = 0; i < n; ++i) Y[i] = logf(X[i]); return 0;
    case KCG_EW_RELU: for (size_t i = 0; i < n; ++i) Y[i] = fmaxf(0.0f, X[i]); return 0;
    case KCG_EW_GELU: for (size_t i = 0; i < n; ++i) Y[i] = oracle_gelu(X[i]); return 0;
    default: return -1;
  }
}

KCG_API void kcg_oracle_gelu_f64(const float *X, double *Y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    double x = (double)X[i];
    double t = tanh((double)(float)0.797884 * ((double)(float)0.044715 * x * x * x + x));
    Y[i] = 0.5 * x * (1.0 + t);
  }
}

/* ------------------------------------------------------------------------ */
/* Attention as the reference graph composes it (test/test.cc:128-130):       */
/* S = BatchedMatmul(Q, K colMajor); P = Softmax(S, last axis, in place);     */
/* O = BatchedMatmul(P, V).  `scale` multiplies S before the softmax and      */
/* `causal` keeps only keys j <= i; scale = 1, causal = 0 is the reference    */
/* graph itself, the other settings reduce to the textbook definition.        */
/* Q,K,V,O are [bh, S, D] row-major with bh = batch*heads flattened.          */
/* The fp32 routine mirrors the three nests op by op (and overflows like the  */
/* reference's max-free softmax would); the fp64 routine is the truth the     */
/* bf16 kernel is measured against.                                           */
/* ------------------------------------------------------------------------ */
KCG_API void kcg_oracle_fmha_f32(const float *Q, const float *K, const float *V, float *O,
                                 int64_t bh, int64_t S, int64_t D, float scale, int causal) {
  float *s = (float *)malloc((size_t)S * sizeof(float));
  for (int64_t b = 0; b < bh; ++b) {
    const float *q_ = Q + b * S * D, *k_ = K + b * S * D, *v_ = V + b * S * D;
    float *o_ = O + b * S * D;
    for (int64_t i = 0; i < S; ++i) {
      const int64_t jn = causal ? i + 1 : S;
      for (int64_t j = 0; j < jn; ++j) {
        float acc = 0.0f;
        for (int64_t d = 0; d < D; ++d) { float mul = q_[i * D + d] * k_[j * D + d]; acc = mul + acc; }
        s[j] = (scale == 1.0f) ? acc : acc * scale;
      }
      float sum = 0.0f;
      for (int64_t j = 0; j < jn; ++j) sum = expf(s[j]) + sum;
      for (int64_t j = 0; j < jn; ++j) s[j] = expf(s[j]) / sum;
      for (int64_t d = 0; d < D; ++d) {
        float acc = 0.0f;
        for (int64_t j = 0; j < jn; ++j) { float mul = s[j] * v_[j * D + d]; acc = mul + acc; }
        o_[i * D + d] = acc;
      }
    }
  }
  free(s);
}

KCG_API void kcg_oracle_fmha_f64(const float *Q, const float *K, const float *V, double *O,
                                 int64_t bh, int64_t S, int64_t D, double scale, int causal) {
  double *s = (double *)malloc((size_t)S * sizeof(double));
  double *acc = (double *)malloc((size_t)D * sizeof(double));
  for (int64_t b = 0; b < bh; ++b) {
    const float *q_ = Q + b * S * D, *k_ = K + b * S * D, *v_ = V + b * S * D;
    double *o_ = O + b * S * D;
    for (int64_t i = 0; i < S; ++i) {
      const int64_t jn = causal ? i + 1 : S;
      double mx = -INFINITY;
      for (int64_t j = 0; j < jn; ++j) {
        double a = 0.0;
        for (int64_t d = 0; d < D; ++d) a += (double)q_[i * D + d] * (double)k_[j * D + d];
        s[j] = a * scale;
        if (s[j] > mx) mx = s[j];
      }
      double sum = 0.0;
      for (int64_t j = 0; j < jn; ++j) { s[j] = exp(s[j] - mx); sum += s[j]; }
      for (int64_t d = 0; d < D; ++d) acc[d] = 0.0;
      for (int64_t j = 0; j < jn; ++j) {
        const double p = s[j] / sum;
        for (int64_t d = 0; d < D; ++d) acc[d] += p * (double)v_[j * D + d];
      }
      for (int64_t d = 0; d < D; ++d) o_[i * D + d] = acc[d];
    }
  }
  free(s);
  free(acc);
}

/* Rows [row0,row0+rows) of one (batch*head) slab, fp64: the bounded sample. */
KCG_API void kcg_oracle_fmha_rows_f64(const float *Q, const float *K, const float *V, double *O,
                                      int64_t S, int64_t D, int64_t row0, int64_t rows,
                                      double scale, int causal) {
  double *s = (double *)malloc((size_t)S * sizeof(double));
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t i = row0 + r;
    const int64_t jn = causal ? i + 1 : S;
    double mx = -INFINITY;
    for (int64_t j = 0; j < jn; ++j) {
      double a = 0.0;
      for (int64_t d = 0; d < D; ++d) a += (double)Q[i * D + d] * (double)K[j * D + d];
      s[j] = a * scale;
      if (s[j] > mx) mx = s[j];
    }
    double sum = 0.0;
    for (int64_t j = 0; j < jn; ++j) { s[j] = exp(s[j] - mx); sum += s[j]; }
    for (int64_t d = 0; d < D; ++d) {
      double a = 0.0;
      for (int64_t j = 0; j < jn; ++j) a += s[j] * (double)V[j * D + d];
      O[r * D + d] = a / sum;
    }
  }
  free(s);
}

/* Relative Frobenius error ||y - ref||_F / ||ref||_F with fp64 reference. */
KCG_API double kcg_oracle_rel_frobenius_f32_f64(const float *y, const double *ref, size_t n) {
  double num = 0.0, den = 0.0;
  for (size_t i = 0; i < n; ++i) {
    double d = (double)y[i] - ref[i];
    num += d * d;
    den += ref[i] * ref[i];
  }
  return den > 0.0 ? sqrt(num / den) : sqrt(num);
}

/* ------------------------------------------------------------------------ */
/* Gather (reference: src/Frontend/Operators.cc:1253-1352): one loop per     */
/* result dimension; out[o, i, r] = in[o, idx[i], r] with o over the dims    */
/* before `axis`, i over the index tensor, r over the dims after it.  Rows   */
/* are moved as bytes, so any element type goes through.  Returns 0, or -1   */
/* when an index is outside [0, axis_extent) (the reference's memref.load    */
/* has no defined result there).                                             */
KCG_API int kcg_oracle_gather(const void* in, const int64_t* idx, void* out, int64_t outer, int64_t axis_extent,
                              int64_t nidx, int64_t row_bytes) {
  const char* src = (const char*)in;
  char* dst = (char*)out;
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t i = 0; i < nidx; ++i) {
      const int64_t j = idx[i];
      if (j < 0 || j >= axis_extent) return -1;
      for (int64_t r = 0; r < row_bytes; ++r)
        dst[(o * nidx + i) * row_bytes + r] = src[(o * axis_extent + j) * row_bytes + r];
    }
  return 0;
}
