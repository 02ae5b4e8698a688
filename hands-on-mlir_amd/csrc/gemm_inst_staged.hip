// Instantiates the staged (any-shape) kernels of the manifest.
#include "gemm_staged.h"
#include "gemm_inst.h"

namespace hom {
namespace gemmk {
#define HOM_INST_STAGED(BM, BN, BK, WM, WN, EPI, VEC)                          \
  template Status launchStaged<BM, BN, BK, WM, WN, EPI, false, VEC>(           \
      const GemmProblem &, hipStream_t);                                       \
  template Status launchStaged<BM, BN, BK, WM, WN, EPI, true, VEC>(            \
      const GemmProblem &, hipStream_t);
#undef HOM_STAGED_TILE
#define HOM_STAGED_TILE(BM, BN, BK, WM, WN, VEC)                               \
  HOM_INST_STAGED(BM, BN, BK, WM, WN, 0, VEC)                                  \
  HOM_INST_STAGED(BM, BN, BK, WM, WN, 1, VEC)                                  \
  HOM_INST_STAGED(BM, BN, BK, WM, WN, 2, VEC)
#include "gemm_manifest.inc"
} // namespace gemmk
} // namespace hom
