/* Source-compatible stand-in for the reference's include/NVGPUKernels/
 * GemmProfiler.h:17-57, the one C++ interface of the kernel library that code
 * outside it uses: the autotune pass constructs a GemmProfiler and calls
 * profile(M, N, K, activation, alpha, beta) for every matmul it meets
 * (lib/Dialect/HOMNVGPU/HOMNVGPUAutotunePass.cpp:85-91), then stores index + 1
 * and the split-K factor on the op.  With this directory ahead of the
 * reference's on the include path and libhom_amdgpu_runner_utils.so in place
 * of GemmManifestAndProfiler on the link line
 * (tools/hands-on-opt/CMakeLists.txt:20), that file compiles unchanged.
 *
 * Header-only over the C entry point homGemmProfile: the timing protocol and
 * the (M, N, K, activation) cache live inside the library, as they do in the
 * reference's GemmProfiler.cu.  The index returned is an index into THIS
 * library's manifest (homGemmManifestName). */
#pragma once

#include "../hom_amdgpu_runner_utils.h"

#include <cstdint>
#include <tuple>

namespace mlir {
namespace hands_on_mlir {
namespace homnvgpu_kernel {

class GemmProfiler {
  int64_t M_, N_, K_, activation_;
  float alpha_, beta_;

public:
  GemmProfiler() = delete;

  GemmProfiler(int64_t M, int64_t N, int64_t K, int64_t activation, float alpha,
               float beta)
      : M_(M), N_(N), K_(K), activation_(activation), alpha_(alpha),
        beta_(beta) {}

  /* (0-based manifest index, split-K factor); index -1 when the nvteGemmF16
   * path is the fastest, as in the reference (GemmProfiler.cu:155-167,225-235),
   * or when no kernel could be timed. */
  std::tuple<int64_t, int32_t> profile() {
    return profile(M_, N_, K_, activation_, alpha_, beta_);
  }

  std::tuple<int64_t, int32_t> profile(int64_t M, int64_t N, int64_t K,
                                       int64_t activation, float alpha,
                                       float beta) {
    int64_t index = -1;
    int32_t splitK = 1;
    homGemmProfile(M, N, K, activation, alpha, beta, &index, &splitK, nullptr);
    return std::make_tuple(index, splitK);
  }
};

} // namespace homnvgpu_kernel
} // namespace hands_on_mlir
} // namespace mlir
