// Host-side runners: memref validation + kernel launch, one per operator of
// the reference's runner classes (include/NVGPUKernels/*Runner.h).  The
// extern "C" entry points in runner_utils.cpp are one-line wrappers over these.
#pragma once

#include "kernels.h"

#include <map>
#include <tuple>
#include <vector>

namespace hom {

// ---- GEMM --------------------------------------------------------------
// Reference-compatible activation codes: 0 linear, 1 GELU.  Extension: 2 asks
// for the tanh form of GELU explicitly (1 means the erf form on the manifest
// path and the tanh form on the nvte path, as in the reference).
Status runGemmManifest(int64_t rankA, void *dstA, int64_t rankB, void *dstB,
                       int64_t rankC, void *dstC, int64_t rankD, void *dstD,
                       int64_t activation, float alpha, float beta,
                       int32_t gemmNum, int32_t splitK, bool noAlloc = false);
Status runGemmNvte(int64_t rankA, void *dstA, bool transa, int64_t rankB,
                   void *dstB, bool transb, int64_t rankC, void *dstC,
                   int64_t rankD, void *dstD, int64_t activation, float alpha,
                   float beta);
Status runGemmWithVarMean(int64_t rankA, void *dstA, int64_t rankB, void *dstB,
                          int64_t rankC, void *dstC, int64_t rankD, void *dstD,
                          int64_t rankVar, void *dstVar, int64_t rankMean,
                          void *dstMean, float alpha, float beta,
                          int64_t activation, float eps);
Status runLayernormGemm(int64_t rankA, void *dstA, int64_t rankB, void *dstB,
                        int64_t rankC, void *dstC, int64_t rankD, void *dstD,
                        int64_t rankVar, void *dstVar, int64_t rankMean,
                        void *dstMean, float alpha, float beta,
                        int64_t activation);

// GEMM with a layer norm (no affine parameters) of the rows of A (mode 1) or
// of C (mode 2) folded in; see launchGemmFolded.
Status runGemmFoldedLayernorm(int64_t rankA, void *dstA, int64_t rankB,
                              void *dstB, int64_t rankC, void *dstC,
                              int64_t rankD, void *dstD, int32_t mode,
                              int64_t activation, float alpha, float beta,
                              const float *statsIn, int32_t piecesIn, float eps,
                              const float *colSumB, float *statsOut,
                              int32_t likeGemmNum);
int32_t foldedLayernormPieces(int64_t M, int64_t N, int64_t K, int64_t activation,
                              int32_t likeGemmNum);
Status runColumnSums(int64_t rankB, void *dstB, float *out);

// Kernel choice without timing: tuned table first, heuristic otherwise.
// `activation`: 0 linear, 1 GELU (erf), 2 GELU (tanh).  Returns true when the
// shape was found in the tuned table.
bool selectGemm(int64_t M, int64_t N, int64_t K, int64_t activation,
                int64_t *idx, int32_t *splitK, bool bIsNK = false);
// What nvteGemmF16 runs for a shape (B as [N, K]; activation 1 is the tanh
// form there), before the per-call alignment fallback.
bool selectGemmNvte(int64_t M, int64_t N, int64_t K, int64_t activation,
                    int64_t *idx, int32_t *splitK);
// Whether the tuned table says that, for this shape, the [N, K] path of
// nvteGemmF16 beats every manifest kernel on row-major B (what the reference's
// profiler reports as index -1).
bool gemmPrefersNvte(int64_t M, int64_t N, int64_t K, int64_t activation);

// Autotuner with the interface of the reference's GemmProfiler
// (include/NVGPUKernels/GemmProfiler.h:20-57).
class GemmProfiler {
public:
  GemmProfiler(int64_t M, int64_t N, int64_t K, int64_t activation, float alpha,
               float beta);
  ~GemmProfiler();
  GemmProfiler(const GemmProfiler &) = delete;
  GemmProfiler &operator=(const GemmProfiler &) = delete;

  // (best 0-based manifest index, best split-K); index -1 = no manifest kernel
  // on row-major B beats the [N, K] path of nvteGemmF16 (the reference's
  // protocol: the compiler then emits nvteGemmF16 for that matmul).
  std::tuple<int64_t, int32_t> profile();
  std::tuple<int64_t, int32_t> profile(int64_t M, int64_t N, int64_t K,
                                       int64_t activation, float alpha,
                                       float beta);
  // Best manifest kernel for one B layout (row-major, or [N, K] when bIsNK),
  // without the baseline; what the table generator asks for.
  std::tuple<int64_t, int32_t> profileLayout(int64_t M, int64_t N, int64_t K,
                                             int64_t activation, float alpha,
                                             float beta, bool bIsNK);
  float bestTimeMs() const { return bestTimeMs_; }

private:
  struct Buffer {
    _Float16 *data = nullptr;
    int64_t capacity = 0; // elements
  };
  bool ensure(Buffer &b, int64_t elems);
  GemmProblem problem(bool bIsNK) const;
  float timeKernel(int idx, int splitK, float previousBest, bool bIsNK);
  void sweep(bool bIsNK, int64_t *bestIdx, int32_t *bestSplit, float *bestTime);
  std::tuple<int64_t, int32_t> run(int mode);

  int64_t M_, N_, K_, activation_;
  float alpha_, beta_;
  float bestTimeMs_ = 0.f;
  Buffer a_, b_, c_;
  hipEvent_t start_ = nullptr, stop_ = nullptr;
  std::map<std::tuple<int64_t, int64_t, int64_t, int64_t>,
           std::tuple<int64_t, int32_t, float>>
      cache_;
};

// ---- other operators ---------------------------------------------------
template <typename T>
Status runLayernorm(int64_t rankA, void *dstA, float eps);
Status runAddLayernormF16(int64_t rankX, void *dstX, int64_t rankRes,
                          void *dstRes, int64_t rankGamma, void *dstGamma,
                          int64_t rankBeta, void *dstBeta, int64_t rankOut,
                          void *dstOut, float eps);
Status runBertAttentionF16(int64_t rankA, void *dstA, int64_t rankSeqlen,
                           void *dstSeqlen, int64_t rankOut, void *dstOut,
                           float scale, int64_t headNum);
template <typename T>
Status runElementwise(BinOp op, int64_t rankA, void *dstA, int64_t rankB,
                      void *dstB, int64_t rankOut, void *dstOut);
template <typename T>
Status runGather(int64_t rankIdx, void *desIdx, int64_t rankValue,
                 void *desValue, int64_t rankOut, void *desOut);
template <typename InT>
Status runCuSeqLen(int64_t rankIn, void *desIn, int64_t rankOut, void *desOut);
Status runGeluF16(int64_t rankA, void *dstA, int64_t rankOut, void *dstOut,
                  int32_t form);

// ---- memory ------------------------------------------------------------
// allocHelper of the reference (HandsOnRunnerUtils.h:46-73) with hipMalloc.
C_UnrankedMemRefType allocDevice(const std::vector<int64_t> &sizes,
                                 size_t elemBytes);
template <typename T> C_UnrankedMemRefType allocConstant(int32_t idx);

} // namespace hom
