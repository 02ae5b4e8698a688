/* CPU oracle for the runtime-kernel path.  TEST INFRASTRUCTURE ONLY: nothing
 * in the product library links, loads or calls this file; it exists so that
 * tests, the smoke check and the benchmark's cpu_baseline leg can check the HIP
 * kernels against an independent restatement of what the reference computes.
 *
 * Every function restates, in plain C with double-precision accumulation, the
 * arithmetic of one operator of the reference's GPU runtime library.  The
 * reference delegates that arithmetic to CUTLASS, TransformerEngine (cuBLASLt,
 * cuDNN) and thrust, none of which are vendored (thirdparty/ is empty,
 * .gitmodules:1-11 names URLs without pins), so each function follows the
 * reference's own call site for shapes, strides and conventions and the
 * operator's published definition for the math:
 *
 *   hom_oracle_gemm          include/NVGPUKernels/GemmRunner.h:244-287 (NN) and
 *                            :328-416 (B as [N,K]); C broadcast rule of
 *                            lib/ExecutionEngine/HandsOnRunnerUtils.cpp:243-266
 *   hom_oracle_gelu_*        erf form = cutlass LinearCombinationGELU
 *                            (python/hom_manifest.py:43-47); tanh form = the
 *                            cuBLASLt epilogue behind GemmRunner.h:386-416;
 *                            polynomial form = include/Conversions/Tosa/
 *                            TosaToHOM.pdll:44-176
 *   hom_oracle_layernorm     include/NVGPUKernels/Layernorm.h:584-694 and the
 *                            pattern include/Conversions/Tosa/TosaToHOM.pdll:19-41
 *   hom_oracle_attention     include/NVGPUKernels/BertAttentionRunner.h:52-136,
 *                            packing lib/Dialect/HOM/HOMFusionPass.cpp:317-346,
 *                            pattern include/Dialect/HOM/HOMFusion.pdll:61-103
 *   hom_oracle_cu_seqlens    include/NVGPUKernels/CuSeqLen.h:48-74
 *   hom_oracle_elementwise   include/NVGPUKernels/ElementwiseRunner.h:69-153
 *   hom_oracle_gather        include/NVGPUKernels/GatherRunner.h:32-77
 *   hom_oracle_row_stats     include/NVGPUKernels/Layernorm.h:33-195 and
 *                            examples/torch/layernorm/cuda/verify.py:72-80
 *   hom_oracle_bert_encoder  call order of lib/Conversions/Function/
 *                            HOMNVGPUToFunc.cpp:76-179,422-470,646-720
 *
 * Parity pinning (see tests/test_oracle.py): every function is checked against
 * the literals the reference's example drivers hold (b.cu, cuSeqLen.cu,
 * layernorm.cu, add.cu, verify.py), against numpy / scipy / torch library
 * routines, and against closed-form identities.  What no reference artefact
 * pins -- cuDNN's output for padded query rows -- is defined here as zeros and
 * is "parity unpinned".
 *
 * fp16 values travel as uint16_t bit patterns; results are returned as float
 * (the "fp32 reference") unless a function says it rounds to fp16.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------- fp16 --- */

ORACLE_API float hom_oracle_half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* float -> half, round to nearest even (what a hardware conversion does). */
ORACLE_API uint16_t hom_oracle_float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u : 0));
  if (absx >= 0x477ff000u) /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  if (absx < 0x33000001u) /* <= 2^-25 rounds to zero */
    return sign;
  int32_t exp = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;
  if (exp < -14) {
    shift = 13 + (-14 - exp); /* subnormal result */
    exp = -15;
  } else {
    shift = 13;
  }
  const uint32_t halfway = 1u << (shift - 1);
  const uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t q = man >> shift;
  if (rem > halfway || (rem == halfway && (q & 1u)))
    q++;
  /* q has the implicit bit at position 10 for normals; adding it to the
   * exponent field carries correctly when rounding overflows the mantissa. */
  uint32_t out = ((uint32_t)(exp + 15) << 10) + q - (exp == -15 ? 0u : 0x400u);
  if (exp == -15)
    out = q; /* subnormal (or smallest normal after carry) */
  return (uint16_t)(sign | out);
}

static inline double h2d(uint16_t h) { return (double)hom_oracle_half_to_float(h); }

/* ---------------------------------------------------------------- GELU --- */

ORACLE_API double hom_oracle_gelu_erf(double x) {
  return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440));
}
ORACLE_API double hom_oracle_gelu_tanh(double x) {
  const double u = 0.79788456080286535588 * (x + 0.044715 * x * x * x);
  return 0.5 * x * (1.0 + tanh(u));
}
/* The decomposed form the TOSA graph carries: erf by Abramowitz-Stegun 7.1.27,
 * erf(t) ~ 1 - 1/(1 + a1 t + a2 t^2 + a3 t^3 + a4 t^4)^4 for t >= 0. */
ORACLE_API double hom_oracle_gelu_poly(double x) {
  const double t = x * 0.707106769;
  const double a = fabs(t);
  const double a2 = a * a, a3 = a2 * a, a4 = a3 * a;
  const double den =
      1.0 + 0.278393 * a + 0.230389 * a2 + 0.000972 * a3 + 0.078108 * a4;
  const double r = 1.0 / den;
  const double r2 = r * r;
  const double e = 1.0 - r2 * r2;
  const double erfv = t >= 0.0 ? e : -e;
  return x * ((erfv + 1.0) * 0.5);
}

static double activate(double v, int act) {
  switch (act) {
  case 1:
    return hom_oracle_gelu_erf(v);
  case 2:
    return hom_oracle_gelu_tanh(v);
  case 3:
    return hom_oracle_gelu_poly(v);
  default:
    return v;
  }
}

/* ---------------------------------------------------------------- GEMM --- */

/* D[m,n] = act(alpha * sum_k A[m,k] B(k,n) + beta * C[(m % c_row_period), n])
 * A [M,K] row-major; B [K,N] row-major, or [N,K] when b_is_nk; C with leading
 * dimension ldc (ignored when beta == 0);
 * act: 0 linear, 1 GELU erf, 2 GELU tanh, 3 GELU polynomial.
 * Inputs are float (fp16 values converted exactly); output D float, unrounded. */
ORACLE_API void hom_oracle_gemm_f32in(const float *A, const float *B,
                                      const float *C, float *D, int64_t M,
                                      int64_t N, int64_t K, int64_t ldc,
                                      int64_t c_row_period, float alpha,
                                      float beta, int act, int b_is_nk) {
  /* B as doubles, K x N, so the inner loop streams */
  double *Bd = (double *)malloc(sizeof(double) * (size_t)(K * N > 0 ? K * N : 1));
  for (int64_t k = 0; k < K; k++)
    for (int64_t n = 0; n < N; n++)
      Bd[k * N + n] = b_is_nk ? (double)B[n * K + k] : (double)B[k * N + n];
  if (c_row_period < 1)
    c_row_period = 1;
#pragma omp parallel
  {
    double *acc = (double *)malloc(sizeof(double) * (size_t)(N > 0 ? N : 1));
#pragma omp for schedule(static)
    for (int64_t m = 0; m < M; m++) {
      for (int64_t n = 0; n < N; n++)
        acc[n] = 0.0;
      for (int64_t k = 0; k < K; k++) {
        const double a = (double)A[m * K + k];
        const double *brow = Bd + k * N;
        for (int64_t n = 0; n < N; n++)
          acc[n] += a * brow[n];
      }
      for (int64_t n = 0; n < N; n++) {
        double v = (double)alpha * acc[n];
        if (beta != 0.0f)
          v += (double)beta * (double)C[(m % c_row_period) * ldc + n];
        D[m * N + n] = (float)activate(v, act);
      }
    }
    free(acc);
  }
  free(Bd);
}

static float *halves_to_floats(const uint16_t *h, int64_t n) {
  if (!h)
    return NULL;
  float *f = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  for (int64_t i = 0; i < n; i++)
    f[i] = hom_oracle_half_to_float(h[i]);
  return f;
}

/* Same with fp16 operands (bit patterns). */
ORACLE_API void hom_oracle_gemm(const uint16_t *A, const uint16_t *B,
                                const uint16_t *C, float *D, int64_t M,
                                int64_t N, int64_t K, int64_t ldc,
                                int64_t c_row_period, float alpha, float beta,
                                int act, int b_is_nk) {
  if (c_row_period < 1)
    c_row_period = 1;
  float *a = halves_to_floats(A, M * K), *b = halves_to_floats(B, K * N);
  float *c = beta != 0.0f ? halves_to_floats(C, (c_row_period - 1) * ldc + N)
                          : NULL;
  hom_oracle_gemm_f32in(a, b, c, D, M, N, K, ldc, c_row_period, alpha, beta, act,
                        b_is_nk);
  free(a);
  free(b);
  free(c);
}

/* ----------------------------------------------------------- LayerNorm --- */

/* out[r,:] = (v - mean(v)) / sqrt(var(v) + eps) * gamma + beta with
 * v = x[r,:] (+ res[r,:]); biased variance.  res/gamma/beta may be NULL.
 * out may alias x. */
ORACLE_API void hom_oracle_layernorm_f32in(const float *x, const float *res,
                                           const float *gamma,
                                           const float *beta, float *out,
                                           int64_t rows, int64_t hidden,
                                           float eps) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; r++) {
    double sum = 0.0;
    for (int64_t j = 0; j < hidden; j++) {
      double v = x[r * hidden + j];
      if (res)
        v += res[r * hidden + j];
      sum += v;
    }
    const double mean = sum / (double)hidden;
    double sq = 0.0;
    for (int64_t j = 0; j < hidden; j++) {
      double v = x[r * hidden + j];
      if (res)
        v += res[r * hidden + j];
      sq += (v - mean) * (v - mean);
    }
    const double rstd = 1.0 / sqrt(sq / (double)hidden + (double)eps);
    for (int64_t j = 0; j < hidden; j++) {
      double v = x[r * hidden + j];
      if (res)
        v += res[r * hidden + j];
      double y = (v - mean) * rstd;
      if (gamma)
        y *= gamma[j];
      if (beta)
        y += beta[j];
      out[r * hidden + j] = (float)y;
    }
  }
}

ORACLE_API void hom_oracle_layernorm_f16(const uint16_t *x, const uint16_t *res,
                                         const uint16_t *gamma,
                                         const uint16_t *beta, float *out,
                                         int64_t rows, int64_t hidden,
                                         float eps) {
  float *xf = halves_to_floats(x, rows * hidden),
        *rf = halves_to_floats(res, rows * hidden),
        *gf = halves_to_floats(gamma, hidden), *bf = halves_to_floats(beta, hidden);
  hom_oracle_layernorm_f32in(xf, rf, gf, bf, out, rows, hidden, eps);
  free(xf);
  free(rf);
  free(gf);
  free(bf);
}

ORACLE_API void hom_oracle_layernorm_f32(const float *x, float *out,
                                         int64_t rows, int64_t hidden,
                                         float eps) {
  for (int64_t r = 0; r < rows; r++) {
    double sum = 0.0, sq = 0.0;
    for (int64_t j = 0; j < hidden; j++)
      sum += x[r * hidden + j];
    const double mean = sum / (double)hidden;
    for (int64_t j = 0; j < hidden; j++)
      sq += (x[r * hidden + j] - mean) * (x[r * hidden + j] - mean);
    const double rstd = 1.0 / sqrt(sq / (double)hidden + (double)eps);
    for (int64_t j = 0; j < hidden; j++)
      out[r * hidden + j] = (float)((x[r * hidden + j] - mean) * rstd);
  }
}

/* Row statistics in the form the LN-GEMM pair exchanges:
 * var[r] = 1/sqrt(E[x^2] - E[x]^2 + eps), mean[r] = -E[x] * var[r]. */
ORACLE_API void hom_oracle_row_stats(const float *d, float *var, float *mean,
                                     int64_t rows, int64_t n, float eps) {
  for (int64_t r = 0; r < rows; r++) {
    double s = 0.0, sq = 0.0;
    for (int64_t j = 0; j < n; j++) {
      s += d[r * n + j];
      sq += (double)d[r * n + j] * d[r * n + j];
    }
    const double m = s / (double)n, ms = sq / (double)n;
    const double v2 = ms - m * m; /* clamped: cancellation on constant rows */
    const double rstd = 1.0 / sqrt((v2 > 0.0 ? v2 : 0.0) + (double)eps);
    var[r] = (float)rstd;
    mean[r] = (float)(-m * rstd);
  }
}

/* ----------------------------------------------------------- attention --- */

/* qkv [bs, seq, 3, heads, d] fp16; cu int32[bs+1]; out [bs, seq, heads, d]
 * float.  Keys >= len_b are masked; query rows >= len_b produce zeros. */
ORACLE_API void hom_oracle_attention_f32in(const float *qkv, const int32_t *cu,
                                           float *out, int64_t bs, int64_t seq,
                                           int64_t heads, int64_t d,
                                           float scale) {
  const int64_t tok = 3 * heads * d;
#pragma omp parallel
  {
    double *p = (double *)malloc(sizeof(double) * (size_t)(seq > 0 ? seq : 1));
#pragma omp for collapse(2) schedule(static)
    for (int64_t b = 0; b < bs; b++) {
      for (int64_t h = 0; h < heads; h++) {
        int64_t len = cu[b + 1] - cu[b];
        if (len < 0)
          len = 0;
        if (len > seq)
          len = seq;
        const float *base = qkv + b * seq * tok;
        for (int64_t q = 0; q < seq; q++) {
          float *o = out + ((b * seq + q) * heads + h) * d;
          if (q >= len) {
            for (int64_t j = 0; j < d; j++)
              o[j] = 0.0f;
            continue;
          }
          const float *qv = base + q * tok + h * d;
          double mx = -INFINITY;
          for (int64_t k = 0; k < len; k++) {
            const float *kv = base + k * tok + (heads + h) * d;
            double s = 0.0;
            for (int64_t j = 0; j < d; j++)
              s += (double)qv[j] * (double)kv[j];
            p[k] = s * (double)scale;
            if (p[k] > mx)
              mx = p[k];
          }
          double denom = 0.0;
          for (int64_t k = 0; k < len; k++) {
            p[k] = exp(p[k] - mx);
            denom += p[k];
          }
          for (int64_t j = 0; j < d; j++) {
            double acc = 0.0;
            for (int64_t k = 0; k < len; k++)
              acc += p[k] * (double)base[k * tok + (2 * heads + h) * d + j];
            o[j] = (float)(acc / denom);
          }
        }
      }
    }
    free(p);
  }
}

ORACLE_API void hom_oracle_attention(const uint16_t *qkv, const int32_t *cu,
                                     float *out, int64_t bs, int64_t seq,
                                     int64_t heads, int64_t d, float scale) {
  float *f = halves_to_floats(qkv, bs * seq * 3 * heads * d);
  hom_oracle_attention_f32in(f, cu, out, bs, seq, heads, d, scale);
  free(f);
}

/* ---------------------------------------------------------- cu_seqlens --- */

ORACLE_API void hom_oracle_cu_seqlens_i64(const int64_t *mask, int32_t *out,
                                          int64_t bs, int64_t seq) {
  out[0] = 0;
  for (int64_t r = 0; r < bs; r++) {
    int32_t s = 0;
    for (int64_t j = 0; j < seq; j++)
      s += (int32_t)mask[r * seq + j];
    out[r + 1] = out[r] + s;
  }
}
ORACLE_API void hom_oracle_cu_seqlens_i32(const int32_t *mask, int32_t *out,
                                          int64_t bs, int64_t seq) {
  out[0] = 0;
  for (int64_t r = 0; r < bs; r++) {
    int32_t s = 0;
    for (int64_t j = 0; j < seq; j++)
      s += mask[r * seq + j];
    out[r + 1] = out[r] + s;
  }
}

/* --------------------------------------------------------- elementwise --- */

/* Index walk of the reference functor: for output linear index x, coordinate i
 * is (x / out_stride[i]) clamped to b_size[i]-1; B is addressed with
 * b_stride.  op: 0 add, 1 sub, 2 mul, 3 div. */
static int64_t bcast_index(int64_t x, int rank, const int64_t *out_stride,
                           const int64_t *b_size, const int64_t *b_stride) {
  int64_t idx = 0;
  for (int i = 0; i < rank; i++) {
    int64_t c = x / out_stride[i];
    x %= out_stride[i];
    if (c >= b_size[i])
      c = b_size[i] - 1;
    idx += c * b_stride[i];
  }
  return idx;
}

static float apply_op(int op, float a, float b) {
  switch (op) {
  case 0:
    return a + b;
  case 1:
    return a - b;
  case 2:
    return a * b;
  default:
    return a / b;
  }
}

/* fp16: the op is evaluated on the fp16 operands and rounded once to fp16
 * (sum, difference and product of two halves are exact in float, the quotient
 * is correctly rounded in float first). Output: fp16 bit patterns. */
ORACLE_API void hom_oracle_elementwise_f16(int op, const uint16_t *a,
                                           const uint16_t *b, uint16_t *out,
                                           int64_t total, int rank,
                                           const int64_t *out_stride,
                                           const int64_t *b_size,
                                           const int64_t *b_stride) {
  for (int64_t i = 0; i < total; i++) {
    const int64_t j = bcast_index(i, rank, out_stride, b_size, b_stride);
    out[i] = hom_oracle_float_to_half(apply_op(
        op, hom_oracle_half_to_float(a[i]), hom_oracle_half_to_float(b[j])));
  }
}
ORACLE_API void hom_oracle_elementwise_f32(int op, const float *a,
                                           const float *b, float *out,
                                           int64_t total, int rank,
                                           const int64_t *out_stride,
                                           const int64_t *b_size,
                                           const int64_t *b_stride) {
  for (int64_t i = 0; i < total; i++) {
    const int64_t j = bcast_index(i, rank, out_stride, b_size, b_stride);
    out[i] = apply_op(op, a[i], b[j]);
  }
}

/* -------------------------------------------------------------- gather --- */

/* out[i, :] = value[indices[i], :] with rows of row_bytes bytes. */
ORACLE_API void hom_oracle_gather(const int64_t *indices, const void *value,
                                  void *out, int64_t n, int64_t row_bytes) {
  for (int64_t i = 0; i < n; i++)
    memcpy((char *)out + i * row_bytes,
           (const char *)value + indices[i] * row_bytes, (size_t)row_bytes);
}

/* -------------------------------------------------------- BERT encoder --- */

/* Round every value to fp16 and back (what storing the tensor as fp16 does). */
static void round_through_half(float *x, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; i++)
    x[i] = hom_oracle_half_to_float(hom_oracle_float_to_half(x[i]));
}

/* The lowered encoder's call list.  Weights per layer: Wqkv [H,3H], Wo [H,H],
 * W1 [H,F], W2 [F,H] (row-major [K,N]), concatenated layer after layer in that
 * order, fp16.  h: in/out hidden states [rows = bs*seq, H] as float holding
 * fp16-representable values on entry.
 * round_intermediates != 0: every tensor the GPU path stores as fp16 is rounded
 * to fp16 here too (the fp16-boundary-faithful oracle); == 0: intermediates
 * stay unrounded (the pure fp32 reference of the same fp16 weights/inputs).
 * gelu_act: 1 erf, 2 tanh.  On return h holds the final layer norm (rounded
 * only if round_intermediates). */
ORACLE_API void hom_oracle_bert_encoder(float *h, const uint16_t *weights,
                                        const int32_t *cu, int64_t layers,
                                        int64_t bs, int64_t seq, int64_t hidden,
                                        int64_t heads, int64_t ffn, float eps,
                                        int gelu_act, int round_intermediates) {
  const int64_t rows = bs * seq, d = hidden / heads;
  float *qkv = (float *)malloc(sizeof(float) * (size_t)(rows * 3 * hidden));
  float *attn = (float *)malloc(sizeof(float) * (size_t)(rows * hidden));
  float *f = (float *)malloc(sizeof(float) * (size_t)(rows * ffn));
  const float scale = (float)(1.0 / sqrt((double)d));
  const int r = round_intermediates;
  const uint16_t *w = weights;
  for (int64_t l = 0; l < layers; l++) {
    float *wqkv = halves_to_floats(w, hidden * 3 * hidden);
    w += hidden * 3 * hidden;
    float *wo = halves_to_floats(w, hidden * hidden);
    w += hidden * hidden;
    float *w1 = halves_to_floats(w, hidden * ffn);
    w += hidden * ffn;
    float *w2 = halves_to_floats(w, ffn * hidden);
    w += ffn * hidden;
    hom_oracle_gemm_f32in(h, wqkv, NULL, qkv, rows, 3 * hidden, hidden, 0, 1,
                          1.0f, 0.0f, 0, 0);
    if (r) round_through_half(qkv, rows * 3 * hidden);
    hom_oracle_attention_f32in(qkv, cu, attn, bs, seq, heads, d, scale);
    if (r) round_through_half(attn, rows * hidden);
    hom_oracle_gemm_f32in(attn, wo, h, h, rows, hidden, hidden, hidden, rows,
                          1.0f, 1.0f, 0, 0);
    if (r) round_through_half(h, rows * hidden);
    hom_oracle_layernorm_f32in(h, NULL, NULL, NULL, h, rows, hidden, eps);
    if (r) round_through_half(h, rows * hidden);
    hom_oracle_gemm_f32in(h, w1, NULL, f, rows, ffn, hidden, 0, 1, 1.0f, 0.0f,
                          gelu_act, 0);
    if (r) round_through_half(f, rows * ffn);
    hom_oracle_gemm_f32in(f, w2, h, h, rows, hidden, ffn, hidden, rows, 1.0f,
                          1.0f, 0, 0);
    if (r) round_through_half(h, rows * hidden);
    hom_oracle_layernorm_f32in(h, NULL, NULL, NULL, h, rows, hidden, eps);
    if (r && l != layers - 1) round_through_half(h, rows * hidden);
    free(wqkv);
    free(wo);
    free(w1);
    free(w2);
  }
  free(qkv);
  free(attn);
  free(f);
}
