// Instantiates the register-staged pipeline kernels of group D of the manifest.
#include "gemm_pipe.h"
#include "gemm_inst.h"

namespace hom {
namespace gemmk {
#undef HOM_PIPE_TILE_D
#define HOM_PIPE_TILE_D(BM, BN, WM, WN, DIST)                                  \
  HOM_INST_EPILOGUES(launchPipe, BM, BN, WM, WN, DIST)
#include "gemm_manifest.inc"
} // namespace gemmk
} // namespace hom
