// The layer-norm pair of the reference (cutlassGemmWithVarMeanF16 followed by
// cutlassLayernormGemmF16, include/NVGPUKernels/LayernormGemmRunner.h:17-361)
// with the normalisation folded into the two GEMMs' epilogues: the first GEMM's
// epilogue accumulates row statistics of the stored D, the second applies
// var/mean per row through the column sums of B.  Both use the register-staged
// pipeline kernels with the two extra epilogue codes.
#include "gemm_pipe.h"

namespace hom {
namespace {
using namespace gemmk;

// ------------------------------------------------------- layer-norm pair --
// Row-statistic partials [pieces][M] (sum, sum of squares) -> var / mean in the
// form the pair exchanges (Layernorm.h:166-192 of the reference: the second
// moment minus the squared mean, no shift).  Four lanes per row, 16 apart in
// the wavefront so that 16 neighbouring lanes read 16 neighbouring rows; each
// takes every fourth piece, four loads in flight.
__global__ __launch_bounds__(256) void rowStatsFinalizeKernel(
    const float *__restrict__ partials, int pieces, int M, int N, float eps,
    _Float16 *__restrict__ var, _Float16 *__restrict__ mean) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int q = lane / 16;
  const int m = (blockIdx.x * 4 + wave) * 16 + lane % 16;
  const int mc = m < M ? m : M - 1;
  float s = 0.f, sq = 0.f;
  for (int pc = q; pc < pieces; pc += 16) {
    float2v v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int pu = pc + 4 * u;
      v[u] = pu < pieces ? *reinterpret_cast<const float2v *>(
                               partials + (int64_t(pu) * M + mc) * 2)
                         : float2v{0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      s += v[u][0];
      sq += v[u][1];
    }
  }
  s = pairSum(rowPairSum(s));
  sq = pairSum(rowPairSum(sq));
  if (q == 0 && m < M) {
    const float mu = s / float(N);
    // the difference cancels to a small negative number for near-constant
    // rows; clamped so that a tiny eps cannot turn it into a NaN
    const float rstd = 1.0f / sqrtf(fmaxf(sq / float(N) - mu * mu, 0.f) + eps);
    var[m] = _Float16(rstd);
    mean[m] = _Float16(-mu * rstd);
  }
}

// Partial column sums of row-major B [K, N]: workgroup (x, y) sums rows
// [y * kPer, (y + 1) * kPer) of columns [32 x, 32 x + 32) into out[y][n].  A
// thread reads 8 columns of every 64th row; the 64 row phases meet in LDS.
__global__ __launch_bounds__(256) void colSumKernel(
    const _Float16 *__restrict__ B, int64_t ldb, int K, int N, int kPer,
    float *__restrict__ out) {
  __shared__ float part[64][33];
  const int tid = threadIdx.x;
  const int cg = tid % 4, ph = tid / 4;
  const int n = blockIdx.x * 32 + cg * 8;
  const int kBegin = blockIdx.y * kPer;
  const int kEnd = kBegin + kPer < K ? kBegin + kPer : K;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (n < N) {
#pragma unroll 4
    for (int k = kBegin + ph; k < kEnd; k += 64) {
      const half8 v = *reinterpret_cast<const half8 *>(B + int64_t(k) * ldb + n);
#pragma unroll
      for (int e = 0; e < 8; e++)
        acc[e] += float(v[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    part[ph][cg * 8 + e] = acc[e];
  __syncthreads();
  // 64 phases -> 8 -> 1, every thread busy in the first step
  {
    const int c = tid % 32, grp = tid / 32;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; r++)
      sum += part[grp * 8 + r][c];
    __syncthreads();
    part[grp][c] = sum;
  }
  __syncthreads();
  if (tid < 32 && blockIdx.x * 32 + tid < N) {
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; r++)
      sum += part[r][tid];
    out[int64_t(blockIdx.y) * N + blockIdx.x * 32 + tid] = sum;
  }
}

// Tiles the layer-norm pair kernels exist in (square, `edge` on a side, a
// wavefront covering `pieceWidth` columns); `likeKernel` picks the nearest.
struct FusedTile {
  int edge;
  int pieceWidth;
};
FusedTile fusedTileFor(int likeKernel) {
  const GemmKernelInfo &like = gemmKernelInfo(likeKernel);
  const int area = like.tileM * like.tileN;
  if (area >= 256 * 256)
    return {256, 64};
  if (area >= 128 * 128)
    return {128, 32};
  return {64, 32};
}
template <int EPI>
Status launchFusedTile(int likeKernel, const GemmProblem &p, hipStream_t s) {
  // the folded-layer-norm epilogues run on the DMA-staged variants of the two
  // smaller tiles (the faster ones at the sizes those tiles serve)
  constexpr bool kDma = EPI >= kEpiFoldA;
  switch (fusedTileFor(likeKernel).edge) {
  case 256:
    return launchPipe<256, 256, 2, 4, 1, EPI, false>(p, s);
  case 128:
    return launchPipe<128, 128, 2, 4, kDma ? 3 : 2, EPI, false, kDma>(p, s);
  default:
    return launchPipe<64, 64, 2, 2, kDma ? 3 : 2, EPI, false, kDma>(p, s);
  }
}

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

} // namespace

bool fusedGemmFits(const GemmProblem &p) {
  return !p.bIsNK && p.M > 0 && p.N > 0 && p.K > 0 &&
         p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31) &&
         p.K < (int64_t(1) << 31) && p.K % 8 == 0 && p.N % 8 == 0 &&
         p.lda % 8 == 0 && p.ldb % 8 == 0 && p.ldd % 8 == 0 &&
         aligned16(p.A) && aligned16(p.B) && aligned16(p.D) &&
         (p.beta == 0.f || (p.C && p.ldc % 8 == 0 && aligned16(p.C)));
}

Status launchGemmRowStats(int likeKernel, const GemmProblem &p, _Float16 *var,
                          _Float16 *mean, float eps, hipStream_t s) {
  HOM_CHECK_RET(likeKernel >= 0 && likeKernel < gemmKernelCount() && fusedGemmFits(p),
                Status::kInvalidArgument,
                "gemm + row statistics: problem does not fit the fused kernels");
  // every tile writes all of its wavefront columns, also those past N
  const FusedTile t = fusedTileFor(likeKernel);
  const int pieces =
      int((p.N + t.edge - 1) / t.edge) * (t.edge / t.pieceWidth);
  float *partials = static_cast<float *>(
      libraryScratch(kTemp, size_t(pieces) * size_t(p.M) * 2 * sizeof(float), false));
  if (!partials)
    return Status::kInternal;
  GemmProblem q = p;
  q.splitK = 1;
  q.rowStatPartials = partials;
  Status st = launchFusedTile<kEpiRowStats>(likeKernel, q, s);
  if (st != Status::kSuccess)
    return st;
  rowStatsFinalizeKernel<<<dim3((unsigned)((p.M + 63) / 64)), dim3(256), 0,
                           s>>>(partials, pieces, int(p.M), int(p.N), eps, var,
                                mean);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

Status launchGemmRowAffine(int likeKernel, const GemmProblem &p,
                           const _Float16 *var, const _Float16 *mean,
                           hipStream_t s) {
  HOM_CHECK_RET(likeKernel >= 0 && likeKernel < gemmKernelCount() && fusedGemmFits(p),
                Status::kInvalidArgument,
                "layernorm + gemm: problem does not fit the fused kernels");
  // 128 rows of B per column-sum workgroup (two 16-byte loads per lane), at
  // most 16 slices
  int slices = int((p.K + 127) / 128);
  if (slices > 16)
    slices = 16;
  const int kPer = int((p.K + slices - 1) / slices);
  float *colSum = static_cast<float *>(
      libraryScratch(kTemp, size_t(slices) * size_t(p.N) * sizeof(float), false));
  if (!colSum)
    return Status::kInternal;
  colSumKernel<<<dim3((unsigned)((p.N + 31) / 32), (unsigned)slices), dim3(256),
                 0, s>>>(p.B, p.ldb, int(p.K), int(p.N), kPer, colSum);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  GemmProblem q = p;
  q.splitK = 1;
  q.rowScale = var;
  q.rowShift = mean;
  q.colSum = colSum;
  q.colSumSlices = slices;
  return launchFusedTile<kEpiRowAffine>(likeKernel, q, s);
}

int foldedPieces(int likeKernel, int64_t N) {
  // one piece per tile column (the wavefront columns of a tile are added up
  // inside the workgroup)
  const FusedTile t = fusedTileFor(likeKernel);
  return int((N + t.edge - 1) / t.edge);
}

Status launchColumnSums(const _Float16 *B, int64_t ldb, int64_t K, int64_t N,
                        float *out, hipStream_t s) {
  HOM_CHECK_RET(K > 0 && N > 0 && K < (int64_t(1) << 31) &&
                    N < (int64_t(1) << 31) && N % 8 == 0 && ldb % 8 == 0 &&
                    aligned16(B),
                Status::kInvalidArgument,
                "column sums: N and the leading dimension must be multiples of 8");
  colSumKernel<<<dim3((unsigned)((N + 31) / 32), 1), dim3(256), 0, s>>>(
      B, ldb, int(K), int(N), int(K), out);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

Status launchGemmFolded(int likeKernel, const GemmProblem &p, int mode,
                        int activation, float *statsOut, hipStream_t s) {
  HOM_CHECK_RET(likeKernel >= 0 && likeKernel < gemmKernelCount() &&
                    fusedGemmFits(p) &&
                    (p.beta == 0.f || (p.cRowPeriod >= p.M && p.ldc % 8 == 0)),
                Status::kInvalidArgument,
                "folded layer norm + gemm: problem does not fit the fused kernels");
  HOM_CHECK_RET((mode == 1 && (activation == 0 || activation == 1) && !statsOut &&
                 (!p.foldStats || p.colSum)) ||
                    (mode == 2 && activation == 0 &&
                     (!p.foldStats || p.beta != 0.f)),
                Status::kInvalidArgument,
                "folded layer norm + gemm: mode %d / activation %d not supported",
                mode, activation);
  // 32-bit byte offsets inside a tile's rows
  HOM_CHECK_RET(int64_t(256) * p.ldd * 2 < (int64_t(1) << 31) &&
                    int64_t(256) * p.ldc * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument,
                "folded layer norm + gemm: leading dimension too large");
  GemmProblem q = p;
  q.splitK = 1;
  q.colSumSlices = 1;
  q.rowStatPartials = statsOut;
  if (mode == 1)
    return activation == 1 ? launchFusedTile<kEpiFoldAGelu>(likeKernel, q, s)
                           : launchFusedTile<kEpiFoldA>(likeKernel, q, s);
  if (!statsOut) {
    // the kernel always writes its partial sums: give it somewhere to put them
    const size_t bytes =
        size_t(foldedPieces(likeKernel, p.N)) * size_t(p.M) * 2 * sizeof(float);
    q.rowStatPartials = static_cast<float *>(libraryScratch(kTemp, bytes, false));
    if (!q.rowStatPartials)
      return Status::kInternal;
  }
  return launchFusedTile<kEpiFoldCStats>(likeKernel, q, s);
}

} // namespace hom
