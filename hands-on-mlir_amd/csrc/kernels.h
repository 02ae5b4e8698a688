// Launch interfaces of the HIP kernels (device pointers + plain sizes).  The
// runners in runners.cpp validate memref arguments and call these.
#pragma once

#include "common.h"

namespace hom {

// ------------------------------------------------------------- layernorm --
// out[r, :] = ((x[r,:] (+ res[r,:])) - mean) * rstd (* gamma + beta).
// T is _Float16 or float.  res/gamma/beta may be null.  out may alias x.
template <typename T>
Status launchLayernorm(const T *x, const T *res, const T *gamma, const T *beta,
                       T *out, int64_t rows, int64_t hidden, float eps,
                       hipStream_t s);

// ----------------------------------------------------------- elementwise --
enum class BinOp : int { kAdd = 0, kSub = 1, kMul = 2, kDiv = 3 };
constexpr int kMaxRank = 8;
struct BroadcastDesc {
  int rank;
  int64_t outSize[kMaxRank];
  int64_t outStride[kMaxRank]; // contiguous strides of A/Out
  int64_t bSize[kMaxRank];
  int64_t bStride[kMaxRank];
};
template <typename T>
Status launchElementwise(BinOp op, const T *a, const T *b, T *out,
                         int64_t total, const BroadcastDesc &desc,
                         hipStream_t s);

template <typename T>
Status launchGather(const int64_t *indices, const T *value, T *out,
                    int64_t numIndices, int64_t vocab, int64_t rowLength,
                    hipStream_t s);

template <typename InT>
Status launchCuSeqLen(const InT *mask, int32_t *out, int64_t bs, int64_t seq,
                      hipStream_t s);

Status launchGeluF16(const _Float16 *in, _Float16 *out, int64_t total, int form,
                     hipStream_t s);

// Per-row statistics of a [rows, n] fp16 matrix in the form the LN-GEMM pair
// exchanges: var[r] = 1/sqrt(E[x^2]-E[x]^2+eps), mean[r] = -E[x]*var[r].
Status launchRowStatsF16(const _Float16 *d, _Float16 *var, _Float16 *mean,
                         int64_t rows, int64_t n, float eps, hipStream_t s);
// out[r, k] = a[r, k] * var[r] + mean[r]  (fp32 math, fp16 store).
Status launchApplyRowStatsF16(const _Float16 *a, const _Float16 *var,
                              const _Float16 *mean, _Float16 *out, int64_t rows,
                              int64_t k, hipStream_t s);

// ------------------------------------------------------------- attention --
// qkv [bs, seq, 3*heads*headDim] fp16, cu int32[bs+1], out [bs, seq,
// heads*headDim].  headDim 64, 128, 192 or 256.
Status launchBertAttentionF16(const _Float16 *qkv, const int32_t *cuSeqlens,
                              _Float16 *out, int64_t bs, int64_t seq,
                              int64_t heads, int64_t headDim, float scale,
                              hipStream_t s);

// ------------------------------------------------------------------ gemm --
enum class Epilogue : int { kLinear = 0, kGeluErf = 1, kGeluTanh = 2 };

struct GemmProblem {
  const _Float16 *A; // [M, K], row stride lda
  const _Float16 *B; // [K, N] row-major (bIsNK false) or [N, K] (bIsNK true)
  const _Float16 *C; // may be null when beta == 0
  _Float16 *D;
  int64_t M, N, K;
  int64_t lda, ldb, ldd;
  // Source addressing: C[(row % cRowPeriod) * ldc + col]; cRowPeriod == M for a
  // full matrix, 1 for a bias row, M' for a per-batch broadcast.  ldc == 0 for
  // a bias row.
  int64_t ldc;
  int64_t cRowPeriod;
  float alpha, beta;
  bool bIsNK;
  int splitK;
  // Split-K partial tiles: null = the library's grow-only scratch (allocated
  // on demand); otherwise a caller-owned device buffer of workspaceBytes that
  // must be large enough (the launch fails instead of allocating).
  float *workspace;
  size_t workspaceBytes;
  // Layer-norm pair, used by launchGemmRowStats / launchGemmRowAffine only
  // (null otherwise).
  // Out: (sum, sum of squares) of every stored row piece, one float2 per row
  // and per wavefront column of the tile grid, [pieces][M].
  float *rowStatPartials;
  // In: D = alpha * (rowScale[m] * (A B)[m,n] + rowShift[m] * colSum[n]) +
  // beta * C, i.e. the product of the row-normalised A with B without ever
  // forming the normalised A.  colSum holds colSumSlices partial column sums
  // of B, [slices][N].
  const _Float16 *rowScale;
  const _Float16 *rowShift;
  const float *colSum;
  int colSumSlices;
  // Folded layer norm, used by launchGemmFolded only (null otherwise): the
  // partial (sum, sum of squares) pairs [foldPieces][M] of the rows that a
  // layer norm is folded away from, 1 / their length, the epsilon.
  const float *foldStats;
  int foldPieces;
  float foldInvN, foldEps;
};

struct GemmKernelInfo {
  const char *name;
  int tileM, tileN, tileK;
  int wavesM, wavesN;
  int alignment; // required divisor of K (8: vector accesses, 1: any shape)
  // Required divisor of N and of the leading dimensions of B (row-major), C, D
  // (8, 2 or 1).  2: rows of B / C / D start at any 4-byte boundary, e.g. the
  // 30522-wide vocabulary projection; the reference's manifest carries separate
  // alignment 8/4/2/1 kernels for this (python/gemm_generator.py:237-278).
  int alignmentN;
  int activation; // 0 linear, 1 gelu (what the profiler filters on)
  Epilogue epilogue;
};

int gemmKernelCount();
const GemmKernelInfo &gemmKernelInfo(int idx);
// Validates alignment/split-K against the kernel and launches it.
Status launchGemm(int idx, const GemmProblem &p, hipStream_t s);
// Device address and size of the fixed split-K scratch array of the current
// device (looked up on the first call per device; never allocates).
Status noAllocWorkspace(float **ptr, size_t *bytes);

// The layer-norm pair with the normalisation folded into the two GEMMs'
// epilogues.  Both need the vector alignment class (K, N and the leading
// dimensions multiples of 8, B row-major) -- fusedGemmFits() says whether a
// problem qualifies -- and `likeKernel`, a manifest index whose tile size they
// imitate.
bool fusedGemmFits(const GemmProblem &p);
// D = alpha A B + beta C, plus per-row statistics of the stored D:
// var[m] = 1 / sqrt(E[d^2] - E[d]^2 + eps), mean[m] = -E[d] * var[m]
// (the statistic is accumulated in the epilogue, a second small kernel turns
// the per-tile partial sums into var / mean).
Status launchGemmRowStats(int likeKernel, const GemmProblem &p, _Float16 *var,
                          _Float16 *mean, float eps, hipStream_t s);
// D = alpha (A * var[m] + mean[m]) B + beta C, computed as
// alpha (var[m] (A B) + mean[m] colsum(B)) + beta C.
Status launchGemmRowAffine(int likeKernel, const GemmProblem &p,
                           const _Float16 *var, const _Float16 *mean,
                           hipStream_t s);

// A layer norm without affine parameters folded into the GEMMs around it (no
// counterpart in the reference, whose pair exchanges finished fp16 statistics
// through two more kernels).  mode 1: D = act(alpha LN(A) B + beta C), act =
// linear or GELU-erf (activation 0 / 1); mode 2: D = alpha A B + beta LN(C).
// The statistics of the normalised rows arrive as the partial sums an earlier
// launchGemmFolded wrote (p.foldStats / foldPieces / foldInvN / foldEps; null:
// no normalisation); mode 1 also needs the column sums of B (p.colSum, one
// slice, see launchColumnSums).  statsOut != null (mode 2 only): the partial
// sums of the stored D go there, foldedPieces(likeKernel, N) x M pairs.
// Needs the alignment class of fusedGemmFits and C absent or a full matrix.
Status launchGemmFolded(int likeKernel, const GemmProblem &p, int mode,
                        int activation, float *statsOut, hipStream_t s);
int foldedPieces(int likeKernel, int64_t N);
// out[n] = sum over k of B[k, n] (fp32), B row-major [K, N], N % 8 == 0.
Status launchColumnSums(const _Float16 *B, int64_t ldb, int64_t K, int64_t N,
                        float *out, hipStream_t s);

} // namespace hom
