// The GEMM kernel manifest and its launch entry (launchGemm): the table that
// cutlassGemmF16's gemmNum indexes, in the role of the reference's generated
// CUTLASS manifest (include/NVGPUKernels/GemmManifest.h:18-67,
// python/gemm_generator.py:237-278).  The kernels themselves are templates in
// gemm_dma.h / gemm_pipe.h / gemm_staged.h, instantiated in gemm_inst_*.hip.
#include "gemm_dma.h"
#include "gemm_fine.h"
#include "gemm_pipe.h"
#include "gemm_staged.h"

namespace hom {
namespace gemmk {
// Instantiated elsewhere (gemm_inst_*.hip).
#define HOM_EXTERN_EPILOGUES(FN, ...)                                          \
  extern template Status FN<__VA_ARGS__, 0, false>(const GemmProblem &,        \
                                                   hipStream_t);               \
  extern template Status FN<__VA_ARGS__, 0, true>(const GemmProblem &,         \
                                                  hipStream_t);                \
  extern template Status FN<__VA_ARGS__, 1, false>(const GemmProblem &,        \
                                                   hipStream_t);               \
  extern template Status FN<__VA_ARGS__, 1, true>(const GemmProblem &,         \
                                                  hipStream_t);                \
  extern template Status FN<__VA_ARGS__, 2, false>(const GemmProblem &,        \
                                                   hipStream_t);               \
  extern template Status FN<__VA_ARGS__, 2, true>(const GemmProblem &,         \
                                                  hipStream_t);
#define HOM_EXTERN_STAGED(BM, BN, BK, WM, WN, EPI, VEC)                        \
  extern template Status launchStaged<BM, BN, BK, WM, WN, EPI, false, VEC>(    \
      const GemmProblem &, hipStream_t);                                       \
  extern template Status launchStaged<BM, BN, BK, WM, WN, EPI, true, VEC>(     \
      const GemmProblem &, hipStream_t);
#define HOM_DMA_TILE(BM, BN, WM, WN, NS)                                       \
  HOM_EXTERN_EPILOGUES(launchDma, BM, BN, WM, WN, NS)
#define HOM_PIPE_TILE_A(BM, BN, WM, WN, DIST)                                  \
  HOM_EXTERN_EPILOGUES(launchPipe, BM, BN, WM, WN, DIST)
#define HOM_PIPE_TILE_B HOM_PIPE_TILE_A
#define HOM_PIPE_TILE_C HOM_PIPE_TILE_A
#define HOM_PIPE_TILE_D HOM_PIPE_TILE_A
#define HOM_FINE_TILE(BM, BN, WM, WN, DIST)                                    \
  HOM_EXTERN_EPILOGUES(launchFine, BM, BN, WM, WN, DIST)
#define HOM_EXTERN_Q(E, NK, BM, BN, WM, WN, DIST)                              \
  extern template Status launchPipe<BM, BN, WM, WN, DIST, E, NK, true>(        \
      const GemmProblem &, hipStream_t);
#define HOM_PIPE_TILE_Q(BM, BN, WM, WN, DIST)                                  \
  HOM_EXTERN_Q(0, false, BM, BN, WM, WN, DIST)                                 \
  HOM_EXTERN_Q(0, true, BM, BN, WM, WN, DIST)                                  \
  HOM_EXTERN_Q(1, false, BM, BN, WM, WN, DIST)                                 \
  HOM_EXTERN_Q(1, true, BM, BN, WM, WN, DIST)                                  \
  HOM_EXTERN_Q(2, false, BM, BN, WM, WN, DIST)                                 \
  HOM_EXTERN_Q(2, true, BM, BN, WM, WN, DIST)
#define HOM_STAGED_TILE(BM, BN, BK, WM, WN, VEC)                               \
  HOM_EXTERN_STAGED(BM, BN, BK, WM, WN, 0, VEC)                                \
  HOM_EXTERN_STAGED(BM, BN, BK, WM, WN, 1, VEC)                                \
  HOM_EXTERN_STAGED(BM, BN, BK, WM, WN, 2, VEC)
#include "gemm_manifest.inc"
#undef HOM_DMA_TILE
#undef HOM_PIPE_TILE_A
#undef HOM_PIPE_TILE_B
#undef HOM_PIPE_TILE_C
#undef HOM_PIPE_TILE_D
#undef HOM_FINE_TILE
#undef HOM_PIPE_TILE_Q
#undef HOM_STAGED_TILE
} // namespace gemmk

namespace {
using namespace gemmk;

using LaunchFn = Status (*)(const GemmProblem &, hipStream_t);

struct KernelEntry {
  GemmKernelInfo info;
  LaunchFn nn; // B as [K, N]
  LaunchFn nt; // B as [N, K]
};

// Names follow the reference generator's scheme (python/hom_manifest.py:56-74):
// <arch>_<opclass>_<acc><instr>gemm_<type>_<tile>_<K>x<stages>_<warps>_<layout>_
// align<n>_<epilogue>; "linear"/"gelu" in the name is what activation is derived
// from (GemmRunner.h:200-206).
#define HOM_DMA_ENTRY(BM, BN, WM, WN, NS, EPI_ENUM, EPI_STR, ACT)              \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_64x" #NS "_w" #WM  \
     "x" #WN "_nn_align8_" EPI_STR,                                            \
     BM, BN, 64, WM, WN, 8, 8, ACT, EPI_ENUM},                                 \
        launchDma<BM, BN, WM, WN, NS, int(EPI_ENUM), false>,                   \
        launchDma<BM, BN, WM, WN, NS, int(EPI_ENUM), true>                     \
  }
#define HOM_DMA_TILE(BM, BN, WM, WN, NS)                                       \
  HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kLinear, "linear", 0),           \
      HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kGeluErf, "gelu", 1),        \
      HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kGeluTanh, "gelutanh", 1),

// "r<d>" after the LDS stage count marks the register-staged pipeline with d
// slabs of global loads in flight.
#define HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, EPI_ENUM, EPI_STR, ACT)           \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_64x2r" #DIST       \
     "_w" #WM "x" #WN "_nn_align8_" EPI_STR,                                   \
     BM, BN, 64, WM, WN, 8, 2, ACT, EPI_ENUM},                                 \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), false>,                \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), true>                  \
  }
// "q<d>": the same pipeline with slabs staged by buffer_load ... lds into a
// ring of d + 1 LDS buffers (d slabs in flight).
#define HOM_PIPE_Q_ENTRY(BM, BN, WM, WN, DIST, EPI_ENUM, EPI_STR, ACT)         \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_64q" #DIST         \
     "_w" #WM "x" #WN "_nn_align8_" EPI_STR,                                   \
     BM, BN, 64, WM, WN, 8, 2, ACT, EPI_ENUM},                                 \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), false, true>,          \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), true, true>            \
  }
#define HOM_PIPE_TILE_Q(BM, BN, WM, WN, DIST)                                  \
  HOM_PIPE_Q_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kLinear, "linear", 0),      \
      HOM_PIPE_Q_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluErf, "gelu", 1),   \
      HOM_PIPE_Q_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluTanh, "gelutanh",  \
                       1),
#define HOM_PIPE_TILE_A(BM, BN, WM, WN, DIST)                                  \
  HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kLinear, "linear", 0),        \
      HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluErf, "gelu", 1),     \
      HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluTanh, "gelutanh", 1),

#define HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, EPI_ENUM, EPI_STR, ACT, VEC)      \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_" #BK "x2_w" #WM   \
     "x" #WN "_nn_align" #VEC "_" EPI_STR,                                     \
     BM, BN, BK, WM, WN, VEC, VEC, ACT, EPI_ENUM},                             \
        launchStaged<BM, BN, BK, WM, WN, int(EPI_ENUM), false, VEC>,           \
        launchStaged<BM, BN, BK, WM, WN, int(EPI_ENUM), true, VEC>             \
  }
#define HOM_STAGED_TILE(BM, BN, BK, WM, WN, VEC)                               \
  HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kLinear, "linear", 0, VEC),   \
      HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluErf, "gelu", 1,      \
                       VEC),                                                   \
      HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluTanh, "gelutanh", 1, \
                       VEC),
#define HOM_PIPE_TILE_B HOM_PIPE_TILE_A
#define HOM_PIPE_TILE_C HOM_PIPE_TILE_A
#define HOM_PIPE_TILE_D HOM_PIPE_TILE_A

// The 16x16x32-MFMA family ("s16x16x32" in the name); N and the leading
// dimensions of B, C, D must be multiples of 8.
#define HOM_FINE_ENTRY(BM, BN, WM, WN, DIST, EPI_ENUM, EPI_STR, ACT)           \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s16x16x32gemm_f16_" #BM "x" #BN "_64x2r" #DIST       \
     "_w" #WM "x" #WN "_nn_align8_" EPI_STR,                                   \
     BM, BN, 64, WM, WN, 8, 8, ACT, EPI_ENUM},                                 \
        launchFine<BM, BN, WM, WN, DIST, int(EPI_ENUM), false>,                \
        launchFine<BM, BN, WM, WN, DIST, int(EPI_ENUM), true>                  \
  }
#define HOM_FINE_TILE(BM, BN, WM, WN, DIST)                                    \
  HOM_FINE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kLinear, "linear", 0),        \
      HOM_FINE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluErf, "gelu", 1),     \
      HOM_FINE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluTanh, "gelutanh", 1),

// Manifest order is part of the ABI: compiled modules carry indices into it.
// New entries go at the end of gemm_manifest.inc.
const KernelEntry kKernels[] = {
#include "gemm_manifest.inc"
};
constexpr int kNumKernels = sizeof(kKernels) / sizeof(kKernels[0]);

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

// Split-K partial tiles of the entry point that may not allocate
// (homGemmF16NoAlloc): a fixed device array instead of the grow-only buffer.
// Every GPU the library runs on holds its own copy for the life of the
// process.  The name below is only a host-side handle; the device address is
// looked up once per device with hipGetSymbolAddress and kernels get that.
constexpr size_t kNoAllocScratchBytes = size_t(32) << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
void *g_scratchAddress[kMaxDevices] = {};

} // namespace

Status noAllocWorkspace(float **ptr, size_t *bytes) {
  int dev = -1;
  HOM_HIP_RET(hipGetDevice(&dev), Status::kInternal);
  HOM_CHECK_RET(dev >= 0 && dev < kMaxDevices, Status::kInternal,
                "gemm: device ordinal %d not supported (max %d)", dev,
                kMaxDevices - 1);
  if (!g_scratchAddress[dev]) {
    void *p = nullptr;
    HOM_HIP_RET(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), Status::kInternal);
    HOM_CHECK_RET(p != nullptr, Status::kInternal,
                  "gemm: no device address for the fixed scratch array");
    g_scratchAddress[dev] = p;
  }
  *ptr = static_cast<float *>(g_scratchAddress[dev]);
  *bytes = kNoAllocScratchBytes;
  return Status::kSuccess;
}

int gemmKernelCount() { return kNumKernels; }
const GemmKernelInfo &gemmKernelInfo(int idx) { return kKernels[idx].info; }

Status launchGemm(int idx, const GemmProblem &p, hipStream_t s) {
  HOM_CHECK_RET(idx >= 0 && idx < kNumKernels, Status::kInvalidArgument,
                "gemm: kernel index %d outside the manifest (size %d)", idx,
                kNumKernels);
  const KernelEntry &k = kKernels[idx];
  HOM_CHECK_RET(p.M >= 0 && p.N >= 0 && p.K >= 0 &&
                    p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31) &&
                    p.K < (int64_t(1) << 31),
                Status::kInvalidArgument, "gemm: problem size out of range");
  HOM_CHECK_RET(p.splitK >= 1, Status::kInvalidArgument,
                "gemm: split-K factor must be >= 1 (got %d)", p.splitK);
  HOM_CHECK_RET(p.beta == 0.f || p.C != nullptr, Status::kInvalidArgument,
                "gemm: beta != 0 needs a source tensor");
  if (k.info.alignment == 8) {
    // What CUTLASS's can_implement() rejects: misaligned leading dimensions.
    // K-contiguous operands (A, and B given as [N, K]) are read 16 bytes at a
    // time from 16-byte aligned rows; row-major B, C and D follow alignmentN.
    const int an = k.info.alignmentN;
    auto alignedTo = [](const void *q, int bytes) {
      return (reinterpret_cast<uintptr_t>(q) & uintptr_t(bytes - 1)) == 0;
    };
    const bool ok =
        p.K % 8 == 0 && p.lda % 8 == 0 && aligned16(p.A) && p.N % an == 0 &&
        (p.bIsNK ? (p.ldb % 8 == 0 && aligned16(p.B))
                 : (p.ldb % an == 0 && alignedTo(p.B, 2 * an))) &&
        p.ldd % an == 0 && alignedTo(p.D, 2 * an) &&
        (p.beta == 0.f || (p.ldc % an == 0 && alignedTo(p.C, 2 * an)));
    HOM_CHECK_RET(ok, Status::kInvalidArgument,
                  "gemm: kernel %s needs K a multiple of 8, N and the leading "
                  "dimensions of B, C, D multiples of %d, and operands aligned "
                  "to match (M=%lld N=%lld K=%lld)",
                  k.info.name, an, (long long)p.M, (long long)p.N,
                  (long long)p.K);
  }
  if (p.M == 0 || p.N == 0)
    return Status::kSuccess;
  return (p.bIsNK ? k.nt : k.nn)(p, s);
}

} // namespace hom
