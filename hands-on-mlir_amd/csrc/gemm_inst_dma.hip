// Instantiates the LDS-DMA kernels of the manifest.
#include "gemm_dma.h"
#include "gemm_inst.h"

namespace hom {
namespace gemmk {
#undef HOM_DMA_TILE
#define HOM_DMA_TILE(BM, BN, WM, WN, NS)                                       \
  HOM_INST_EPILOGUES(launchDma, BM, BN, WM, WN, NS)
#include "gemm_manifest.inc"
} // namespace gemmk
} // namespace hom
