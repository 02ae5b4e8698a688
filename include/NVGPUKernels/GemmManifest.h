/* Source-compatible stand-in for the reference's include/NVGPUKernels/
 * GemmManifest.h:18-65 (the `manifest` object: an ordered list of GEMM
 * operations indexed by the number a compiled module carries) and for the part
 * of GemmOperationRunnerBase (include/NVGPUKernels/GemmRunner.h:119-138) that
 * code outside the kernel library can use: run(), contains(), isF16(),
 * getActivation() and the operation's name.
 *
 * Header-only over the C entry points of libhom_amdgpu_runner_utils.so: the
 * kernels and their table live inside the library (csrc/gemm_manifest.inc is
 * the list, its order the ABI); this class only presents them with the
 * reference's interface.  manifest[i] is the operation cutlassGemmF16 runs
 * for gemmNum == i + 1.
 *
 * Differences, on purpose: there is no append() / reserve() / initialize_all()
 * (the reference fills its manifest from generated CUTLASS instances at start-up,
 * python/gemm_generator.py:237-278; here the list is fixed at build time), and
 * run() returns 0 on success or a non-zero status instead of cutlass::Status. */
#pragma once

#include "../hom_amdgpu_runner_utils.h"

#include <cstddef>
#include <cstdint>
#include <cstring>

namespace mlir {
namespace hands_on_mlir {
namespace homnvgpu_kernel {

class GemmOperationRunnerBase {
  int32_t index_; /* 0-based manifest index */

public:
  explicit GemmOperationRunnerBase(int32_t index) : index_(index) {}

  const char *getName() const { return homGemmManifestName(index_); }

  /* GemmRunner.h:129: substring test on the operation's name. */
  bool contains(const char *str) const {
    const char *name = getName();
    return name != nullptr && str != nullptr && std::strstr(name, str) != nullptr;
  }

  /* Every manifest kernel computes fp16 operands with fp32 accumulation. */
  bool isF16() const { return true; }

  /* 0 for a "linear" operation, 1 for a "gelu" one (GemmRunner.h:200-206). */
  int32_t getActivation() const { return homGemmManifestActivation(index_); }

  int32_t getAlignment() const { return homGemmManifestAlignment(index_); }

  /* D = act(alpha * A.B + beta * C) through the library's entry point with this
   * operation's number; descriptors as in cutlassGemmF16.  Errors follow the
   * library's error mode (homSetErrorMode): print-and-abort by default, or a
   * recorded message and a non-zero return. */
  int run(int64_t rankA, void *dstA, int64_t rankB, void *dstB, int64_t rankC,
          void *dstC, int64_t rankD, void *dstD, float alpha, float beta,
          int32_t splitKFactor) const {
    cutlassGemmF16(rankA, dstA, false, rankB, dstB, false, rankC, dstC, rankD,
                   dstD, getActivation(), alpha, beta, index_ + 1, splitKFactor);
    const char *err = homGetLastError();
    return err != nullptr && err[0] != '\0' ? 1 : 0;
  }
};

class GemmManifest {
public:
  void updateAllKernels() {}
  void init() {}

  GemmOperationRunnerBase getKernel(int32_t idx) const {
    return GemmOperationRunnerBase(idx);
  }
  GemmOperationRunnerBase operator[](int idx) const {
    return GemmOperationRunnerBase(int32_t(idx));
  }
  size_t size() const { return size_t(homGemmManifestSize()); }

  /* 0-based index of the operation with this name, -1 if there is none. */
  int32_t find(const char *name) const { return homGemmManifestFind(name); }
};

inline GemmManifest manifest;

} // namespace homnvgpu_kernel
} // namespace hands_on_mlir
} // namespace mlir
