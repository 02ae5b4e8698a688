// Instantiates the pipeline kernels that stage slabs with buffer_load ... lds
// (group Q of the manifest).
#include "gemm_pipe.h"
#include "gemm_inst.h"

namespace hom {
namespace gemmk {
#undef HOM_PIPE_TILE_Q
#define HOM_PIPE_TILE_Q(BM, BN, WM, WN, DIST)                                  \
  HOM_INST_EPILOGUES_DMA(launchPipe, BM, BN, WM, WN, DIST)
#include "gemm_manifest.inc"
} // namespace gemmk
} // namespace hom
