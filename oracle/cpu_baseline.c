/* Single-threaded fp32 restatement of what the reference's TOSA -> LLVM CPU
 * lowering executes for the same operators, used only to report a CPU baseline
 * next to the GPU numbers.  TEST / BENCHMARK INFRASTRUCTURE ONLY: the product
 * library never links or calls this.
 *
 *  - GEMM: the loop nest of matmulAddF32 (lib/ExecutionEngine/
 *    HandsOnRunnerUtils.cpp:230-277): copy/broadcast C into D, then
 *    for b, i, j, k: D[b,i,j] += A[i,k] * B[k,j], fp32, that loop order.
 *  - GELU, layer norm, softmax: the decomposed elementwise / reduce graphs the
 *    compiler pattern-matches (include/Conversions/Tosa/TosaToHOM.pdll:6-17
 *    softmax, :19-41 layer norm, :44-176 GELU with the Abramowitz-Stegun erf
 *    polynomial), run as separate passes over fp32 buffers with no fusion, the
 *    way a scalar lowering of those graphs runs.
 *  - attention: Q.K^T, scale, additive mask, softmax, .V as the unfused graph
 *    (include/Dialect/HOM/HOMFusion.pdll:61-103).
 * The reference's generated CPU code has no threading, so neither has this.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BASELINE_API __attribute__((visibility("default")))

BASELINE_API void hom_cpu_matmul_add_f32(const float *A, const float *B,
                                         const float *C, float *D,
                                         int64_t batch, int64_t M, int64_t N,
                                         int64_t K, int c_batch, int c_rows) {
  for (int64_t b = 0; b < batch; b++)
    for (int64_t i = 0; i < M; i++)
      for (int64_t j = 0; j < N; j++)
        D[(b * M + i) * N + j] =
            C ? C[((c_batch == 1 ? 0 : b) * (c_rows == 1 ? 1 : M) +
                   (c_rows == 1 ? 0 : i)) * N + j]
              : 0.0f;
  for (int64_t b = 0; b < batch; b++)
    for (int64_t i = 0; i < M; i++)
      for (int64_t j = 0; j < N; j++) {
        float acc = D[(b * M + i) * N + j];
        for (int64_t k = 0; k < K; k++)
          acc += A[(b * M + i) * K + k] * B[k * N + j];
        D[(b * M + i) * N + j] = acc;
      }
}

/* GELU as the chain of elementwise TOSA ops, one pass per op. */
BASELINE_API void hom_cpu_gelu_tosa_f32(const float *x, float *out, float *t0,
                                        float *t1, int64_t n) {
  for (int64_t i = 0; i < n; i++) t0[i] = x[i] * 0.707106769f;     /* mul   */
  for (int64_t i = 0; i < n; i++) t1[i] = fabsf(t0[i]);            /* abs   */
  for (int64_t i = 0; i < n; i++) {                                /* poly  */
    const float a = t1[i], a2 = a * a, a3 = a2 * a, a4 = a3 * a;
    out[i] = 1.0f + 0.278393f * a + 0.230389f * a2 + 0.000972f * a3 +
             0.078108f * a4;
  }
  for (int64_t i = 0; i < n; i++) out[i] = 1.0f / out[i];          /* recip */
  for (int64_t i = 0; i < n; i++) out[i] = out[i] * out[i];        /* ^2    */
  for (int64_t i = 0; i < n; i++) out[i] = 1.0f - out[i] * out[i]; /* 1-^4  */
  for (int64_t i = 0; i < n; i++)                                  /* select*/
    out[i] = t0[i] >= 0.0f ? out[i] : -out[i];
  for (int64_t i = 0; i < n; i++) out[i] = (out[i] + 1.0f) * 0.5f;
  for (int64_t i = 0; i < n; i++) out[i] = x[i] * out[i];
}

/* Layer norm as reduce_sum, mul, sub, mul, reduce_sum, mul, add, rsqrt, mul. */
BASELINE_API void hom_cpu_layernorm_tosa_f32(float *x, float *tmp,
                                             int64_t rows, int64_t hidden,
                                             float eps) {
  const float inv = 1.0f / (float)hidden;
  for (int64_t r = 0; r < rows; r++) {
    float s = 0.0f;
    for (int64_t j = 0; j < hidden; j++) s += x[r * hidden + j];
    const float mean = s * inv;
    for (int64_t j = 0; j < hidden; j++) tmp[r * hidden + j] = x[r * hidden + j] - mean;
    float sq = 0.0f;
    for (int64_t j = 0; j < hidden; j++) sq += tmp[r * hidden + j] * tmp[r * hidden + j];
    const float rstd = 1.0f / sqrtf(sq * inv + eps);
    for (int64_t j = 0; j < hidden; j++) x[r * hidden + j] = tmp[r * hidden + j] * rstd;
  }
}

BASELINE_API void hom_cpu_add_f32(const float *a, const float *b, float *out,
                                  int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* Unfused attention on fp32 qkv [bs, seq, 3, heads, d]; lens[b] valid keys.
 * scores: scratch [seq, seq]. */
BASELINE_API void hom_cpu_attention_f32(const float *qkv, const int32_t *lens,
                                        float *out, float *scores, int64_t bs,
                                        int64_t seq, int64_t heads, int64_t d,
                                        float scale) {
  const int64_t tok = 3 * heads * d;
  for (int64_t b = 0; b < bs; b++)
    for (int64_t h = 0; h < heads; h++) {
      const float *base = qkv + b * seq * tok;
      for (int64_t q = 0; q < seq; q++)
        for (int64_t k = 0; k < seq; k++) {
          float s = 0.0f;
          for (int64_t j = 0; j < d; j++)
            s += base[q * tok + h * d + j] * base[k * tok + (heads + h) * d + j];
          scores[q * seq + k] = s * scale + (k < lens[b] ? 0.0f : -1e9f);
        }
      for (int64_t q = 0; q < seq; q++) { /* softmax, TOSA decomposition */
        float mx = -INFINITY, sum = 0.0f;
        for (int64_t k = 0; k < seq; k++) mx = fmaxf(mx, scores[q * seq + k]);
        for (int64_t k = 0; k < seq; k++) scores[q * seq + k] = expf(scores[q * seq + k] - mx);
        for (int64_t k = 0; k < seq; k++) sum += scores[q * seq + k];
        const float r = 1.0f / sum;
        for (int64_t k = 0; k < seq; k++) scores[q * seq + k] *= r;
      }
      for (int64_t q = 0; q < seq; q++)
        for (int64_t j = 0; j < d; j++) {
          float acc = 0.0f;
          for (int64_t k = 0; k < seq; k++)
            acc += scores[q * seq + k] * base[k * tok + (2 * heads + h) * d + j];
          out[((b * seq + q) * heads + h) * d + j] = acc;
        }
    }
}
