// Instantiates the 16x16x32-MFMA kernels of the manifest.
#include "gemm_fine.h"
#include "gemm_inst.h"

namespace hom {
namespace gemmk {
#undef HOM_FINE_TILE
#define HOM_FINE_TILE(BM, BN, WM, WN, DIST)                                    \
  HOM_INST_EPILOGUES(launchFine, BM, BN, WM, WN, DIST)
#include "gemm_manifest.inc"
} // namespace gemmk
} // namespace hom
