// extern "C" boundary of libhom_amdgpu_runner_utils.so.  Each entry point has
// the name and signature of the reference's shim
// (lib/ExecutionEngine/HandsOnNVGPURunnerUtils.cu:78-377) and forwards to a
// runner; status handling (abort or record) lives in the HOM_CHECK macros.
#include "hom_amdgpu_runner_utils.h"
#include "runners.h"

#include <cstring>
#include <memory>

using namespace hom;

namespace {
GemmProfiler *g_profiler = nullptr; // never destroyed: HIP may be gone at exit

void printSizes(int64_t rank, void *descriptor) {
  fprintf(stderr, "Print inside: ");
  if (descriptor) {
    const int64_t *sizes = hom_memref_sizes(descriptor);
    for (int64_t i = 0; i < rank; i++)
      fprintf(stderr, "%lld ", (long long)sizes[i]);
  }
  fprintf(stderr, "\n");
}

void freeData(void *descriptor) {
  if (!descriptor)
    return;
  auto *h = static_cast<HomMemRefHeader *>(descriptor);
  if (h->data) {
    hipError_t e = hipFree(h->data);
    if (e != hipSuccess)
      recordError(__FILE__, __LINE__, "dealloc: hipFree failed: %s",
                  hipGetErrorString(e));
  }
}
} // namespace

extern "C" {

// ------------------------------------------------------------------ GEMM --
void cutlassGemmF32(int64_t, void *, bool, int64_t, void *, bool, int64_t,
                    void *, int64_t, void *, int64_t, float, float) {}

void cutlassGemmF16(int64_t rankA, void *dstA, bool transa, int64_t rankB,
                    void *dstB, bool transb, int64_t rankC, void *dstC,
                    int64_t rankD, void *dstD, int64_t activation, float alpha,
                    float beta, int32_t gemmNum, int32_t splitKFactor) {
  (void)transa;
  (void)transb;
  (void)runGemmManifest(rankA, dstA, rankB, dstB, rankC, dstC, rankD, dstD,
                        activation, alpha, beta, gemmNum, splitKFactor);
}

void homGemmF16NoAlloc(int64_t rankA, void *dstA, bool transa, int64_t rankB,
                       void *dstB, bool transb, int64_t rankC, void *dstC,
                       int64_t rankD, void *dstD, int64_t activation,
                       float alpha, float beta, int32_t gemmNum,
                       int32_t splitKFactor) {
  (void)transa;
  (void)transb;
  (void)runGemmManifest(rankA, dstA, rankB, dstB, rankC, dstC, rankD, dstD,
                        activation, alpha, beta, gemmNum, splitKFactor, true);
}

void nvteGemmF16(int64_t rankA, void *dstA, bool transa, int64_t rankB,
                 void *dstB, bool transb, int64_t rankC, void *dstC,
                 int64_t rankD, void *dstD, int64_t activation, float alpha,
                 float beta, int32_t, int32_t) {
  (void)runGemmNvte(rankA, dstA, transa, rankB, dstB, transb, rankC, dstC,
                    rankD, dstD, activation, alpha, beta);
}

void cutlassGemmWithVarMeanF16(int64_t rankA, void *dstA, int64_t rankB,
                               void *dstB, int64_t rankC, void *dstC,
                               int64_t rankD, void *dstD, int64_t rankVar,
                               void *dstVar, int64_t rankMean, void *dstMean,
                               float alpha, float beta, int64_t activation,
                               float eps) {
  (void)runGemmWithVarMean(rankA, dstA, rankB, dstB, rankC, dstC, rankD, dstD,
                           rankVar, dstVar, rankMean, dstMean, alpha, beta,
                           activation, eps);
}

void cutlassLayernormGemmF32(int64_t, void *, int64_t, void *, int64_t, void *,
                             int64_t, void *, int64_t, void *, int64_t, void *,
                             float, float, int64_t) {}

void cutlassLayernormGemmF16(int64_t rankA, void *dstA, int64_t rankB,
                             void *dstB, int64_t rankC, void *dstC,
                             int64_t rankD, void *dstD, int64_t rankVar,
                             void *dstVar, int64_t rankMean, void *dstMean,
                             float alpha, float beta, int64_t activation) {
  (void)runLayernormGemm(rankA, dstA, rankB, dstB, rankC, dstC, rankD, dstD,
                         rankVar, dstVar, rankMean, dstMean, alpha, beta,
                         activation);
}

// ------------------------------------------------------------- layer norm --
void nvteLayernormF32(int64_t rankA, void *dstA, float eps) {
  (void)runLayernorm<float>(rankA, dstA, eps);
}
void nvteLayernormF16(int64_t rankA, void *dstA, float eps) {
  (void)runLayernorm<_Float16>(rankA, dstA, eps);
}

// -------------------------------------------------------------- attention --
void nvteBertAttentionF16(int64_t rankA, void *dstA, int64_t rankSeqlen,
                          void *dstSeqlen, int64_t rankOut, void *dstOut,
                          float scale, int64_t headNum) {
  (void)runBertAttentionF16(rankA, dstA, rankSeqlen, dstSeqlen, rankOut, dstOut,
                            scale, headNum);
}
void nvteBertAttentionF32(int64_t, void *, int64_t, void *, int64_t, void *,
                          float, int64_t) {
  // The reference instantiates BertAttentionRunner<float>, which the fused
  // attention backend it calls rejects at run time (fp16/bf16 only).
  recordError(__FILE__, __LINE__,
              "nvteBertAttentionF32: fp32 attention is not supported");
}

// ------------------------------------------- elementwise / gather / seqlen --
#define HOM_ELEMENTWISE_DEF(op, suffix, type)                                  \
  void thrustElementwise##op##suffix(int64_t rankA, void *dstA, int64_t rankB, \
                                     void *dstB, int64_t rankOut,              \
                                     void *dstOut) {                           \
    (void)runElementwise<type>(BinOp::k##op, rankA, dstA, rankB, dstB,         \
                               rankOut, dstOut);                               \
  }
HOM_ELEMENTWISE_DEF(Add, F32, float)
HOM_ELEMENTWISE_DEF(Sub, F32, float)
HOM_ELEMENTWISE_DEF(Mul, F32, float)
HOM_ELEMENTWISE_DEF(Div, F32, float)
HOM_ELEMENTWISE_DEF(Add, F16, _Float16)
HOM_ELEMENTWISE_DEF(Sub, F16, _Float16)
HOM_ELEMENTWISE_DEF(Mul, F16, _Float16)
HOM_ELEMENTWISE_DEF(Div, F16, _Float16)

void thrustGatherF32(int64_t rankIndices, void *desIndices, int64_t rankValue,
                     void *desValue, int64_t rankOut, void *desOut) {
  (void)runGather<float>(rankIndices, desIndices, rankValue, desValue, rankOut,
                         desOut);
}
void thrustGatherF16(int64_t rankIndices, void *desIndices, int64_t rankValue,
                     void *desValue, int64_t rankOut, void *desOut) {
  (void)runGather<_Float16>(rankIndices, desIndices, rankValue, desValue,
                            rankOut, desOut);
}

void thrustCuSeqLenI64(int64_t rankInput, void *desInput, int64_t rankOut,
                       void *desOut) {
  (void)runCuSeqLen<int64_t>(rankInput, desInput, rankOut, desOut);
}
void thrustCuSeqLenI32(int64_t rankInput, void *desInput, int64_t rankOut,
                       void *desOut) {
  (void)runCuSeqLen<int32_t>(rankInput, desInput, rankOut, desOut);
}

// ----------------------------------------------------------------- memory --
C_UnrankedMemRefType alloc3DMemRefNVGPUF32(int32_t a, int32_t b, int32_t c) {
  return allocDevice({a, b, c}, sizeof(float));
}
C_UnrankedMemRefType alloc3DMemRefNVGPUF16(int32_t a, int32_t b, int32_t c) {
  return allocDevice({a, b, c}, sizeof(_Float16));
}
C_UnrankedMemRefType alloc1DMemRefNVGPUI32(int32_t a) {
  return allocDevice({a}, sizeof(int32_t));
}
C_UnrankedMemRefType allocConstantNVGPUF32(int32_t idx) {
  return allocConstant<float>(idx);
}
C_UnrankedMemRefType allocConstantNVGPUF16(int32_t idx) {
  return allocConstant<_Float16>(idx);
}
void deallocNVGPUF32(int64_t, void *dst) { freeData(dst); }
void deallocNVGPUF16(int64_t, void *dst) { freeData(dst); }
void deallocNVGPUI32(int64_t, void *dst) { freeData(dst); }

// ------------------------------------------------------------------ debug --
void printMemrefSizeF32(int64_t rk, void *d) { printSizes(rk, d); }
void printMemrefSizeF16(int64_t rk, void *d) { printSizes(rk, d); }
void printMemrefSizeI64(int64_t rk, void *d) { printSizes(rk, d); }
void printMemrefSizeI32(int64_t rk, void *d) { printSizes(rk, d); }

// ------------------------------------------------------------- extensions --
void homSetStream(void *hipStream) {
  setStream(static_cast<hipStream_t>(hipStream));
}
void *homGetStream(void) { return static_cast<void *>(stream()); }
void homReleaseStreamScratch(void *hipStream) {
  releaseStreamScratch(static_cast<hipStream_t>(hipStream));
}
void homSetSplitKInKernel(int32_t mode) {
  setSplitKInKernel(mode >= 0 && mode <= 3 ? mode : 3);
}
int32_t homSplitKInKernelLaunches(void) { return splitKInKernelLaunches(); }
void homSetErrorMode(int32_t mode) { setErrorMode(mode == 1 ? 1 : 0); }
const char *homGetLastError(void) { return takeLastError(); }
int32_t homScratchGeneration(void) { return libraryScratchGeneration(); }

void homAddLayernormF16(int64_t rankX, void *dstX, int64_t rankRes,
                        void *dstRes, int64_t rankGamma, void *dstGamma,
                        int64_t rankBeta, void *dstBeta, int64_t rankOut,
                        void *dstOut, float eps) {
  (void)runAddLayernormF16(rankX, dstX, rankRes, dstRes, rankGamma, dstGamma,
                           rankBeta, dstBeta, rankOut, dstOut, eps);
}

void homGemmFoldedLayernormF16(int64_t rankA, void *dstA, int64_t rankB,
                               void *dstB, int64_t rankC, void *dstC,
                               int64_t rankD, void *dstD, int32_t mode,
                               int64_t activation, float alpha, float beta,
                               const float *statsIn, int32_t piecesIn, float eps,
                               const float *colSumB, float *statsOut,
                               int32_t likeGemmNum) {
  (void)runGemmFoldedLayernorm(rankA, dstA, rankB, dstB, rankC, dstC, rankD,
                               dstD, mode, activation, alpha, beta, statsIn,
                               piecesIn, eps, colSumB, statsOut, likeGemmNum);
}

int32_t homFoldedLayernormPieces(int64_t M, int64_t N, int64_t K,
                                 int64_t activation, int32_t likeGemmNum) {
  return foldedLayernormPieces(M, N, K, activation, likeGemmNum);
}

void homColumnSumsF16(int64_t rankB, void *dstB, float *out) {
  (void)runColumnSums(rankB, dstB, out);
}

void homGeluF16(int64_t rankA, void *dstA, int64_t rankOut, void *dstOut,
                int32_t form) {
  (void)runGeluF16(rankA, dstA, rankOut, dstOut, form);
}

int32_t homGemmManifestSize(void) { return gemmKernelCount(); }
const char *homGemmManifestName(int32_t idx) {
  if (idx < 0 || idx >= gemmKernelCount())
    return "";
  return gemmKernelInfo(idx).name;
}
int32_t homGemmManifestActivation(int32_t idx) {
  if (idx < 0 || idx >= gemmKernelCount())
    return -1;
  return gemmKernelInfo(idx).activation;
}
int32_t homGemmManifestAlignment(int32_t idx) {
  if (idx < 0 || idx >= gemmKernelCount())
    return -1;
  return gemmKernelInfo(idx).alignment;
}
int32_t homGemmManifestFind(const char *name) {
  if (!name)
    return -1;
  for (int i = 0; i < gemmKernelCount(); i++)
    if (strcmp(gemmKernelInfo(i).name, name) == 0)
      return i;
  return -1;
}

void homGemmProfile(int64_t M, int64_t N, int64_t K, int64_t activation,
                    float alpha, float beta, int64_t *bestIdx,
                    int32_t *bestSplitK, float *bestTimeMs) {
  if (!g_profiler)
    g_profiler = new GemmProfiler(M, N, K, activation, alpha, beta);
  auto res = g_profiler->profile(M, N, K, activation, alpha, beta);
  if (bestIdx)
    *bestIdx = std::get<0>(res);
  if (bestSplitK)
    *bestSplitK = std::get<1>(res);
  if (bestTimeMs)
    *bestTimeMs = g_profiler->bestTimeMs();
}

void homGemmProfileLayout(int64_t M, int64_t N, int64_t K, int64_t activation,
                          float alpha, float beta, int32_t bIsNK,
                          int64_t *bestIdx, int32_t *bestSplitK,
                          float *bestTimeMs) {
  if (!g_profiler)
    g_profiler = new GemmProfiler(M, N, K, activation, alpha, beta);
  auto res =
      g_profiler->profileLayout(M, N, K, activation, alpha, beta, bIsNK != 0);
  if (bestIdx)
    *bestIdx = std::get<0>(res);
  if (bestSplitK)
    *bestSplitK = std::get<1>(res);
  if (bestTimeMs)
    *bestTimeMs = g_profiler->bestTimeMs();
}

int32_t homGemmSelect(int64_t M, int64_t N, int64_t K, int64_t activation,
                      int64_t *idx, int32_t *splitK) {
  int64_t i = -1;
  int32_t s = 1;
  const bool tuned = selectGemm(M, N, K, activation, &i, &s);
  if (idx)
    *idx = i;
  if (splitK)
    *splitK = s;
  return tuned ? 1 : 0;
}

int32_t homGemmSelectNvte(int64_t M, int64_t N, int64_t K, int64_t activation,
                          int64_t *idx, int32_t *splitK) {
  int64_t i = -1;
  int32_t s = 1;
  const bool tuned = selectGemmNvte(M, N, K, activation, &i, &s);
  if (idx)
    *idx = i;
  if (splitK)
    *splitK = s;
  return tuned ? 1 : 0;
}

int32_t homGemmPrefersNvte(int64_t M, int64_t N, int64_t K, int64_t activation) {
  return gemmPrefersNvte(M, N, K, activation) ? 1 : 0;
}

} // extern "C"
