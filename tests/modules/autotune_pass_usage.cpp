// The part of the reference's autotune pass that touches the kernel library
// (lib/Dialect/HOMNVGPU/HOMNVGPUAutotunePass.cpp:52-92), without the MLIR
// types around it: same include, same namespace, same calls.  Built by
// tests/test_abi.py against include/NVGPUKernels/GemmProfiler.h and
// libhom_amdgpu_runner_utils.so; with "run" as its argument it profiles one
// shape on the GPU and prints the result.
#include "NVGPUKernels/GemmManifest.h"
#include "NVGPUKernels/GemmProfiler.h"

#include <cstdio>
#include <cstring>

namespace {
struct MatmulOpStandIn {
  int64_t kernelName = 0;
  int32_t splitK = 0;
  void setKernelName(int64_t v) { kernelName = v; }
  void setSplitKFactor(int32_t v) { splitK = v; }
};

void profileMatmulImpl(MatmulOpStandIn &gemm, int64_t M, int64_t N, int64_t K,
                       int64_t act, float alpha, float beta) {
  using namespace mlir::hands_on_mlir::homnvgpu_kernel;
  static GemmProfiler profiler(M, N, K, act, alpha, beta);
  auto [bestIdx, bestSplitKFactor] = profiler.profile(M, N, K, act, alpha, beta);
  gemm.setKernelName(bestIdx + 1);
  gemm.setSplitKFactor(bestSplitKFactor);
}
} // namespace

int main(int argc, char **argv) {
  if (argc > 1 && strcmp(argv[1], "run") == 0) {
    MatmulOpStandIn op;
    profileMatmulImpl(op, 256, 768, 768, 0, 1.0f, 0.0f);
    printf("%lld %d %s\n", (long long)op.kernelName, op.splitK,
           op.kernelName >= 1 ? homGemmManifestName(int32_t(op.kernelName - 1))
                              : "nvte");
    // kernel number 0 = the nvteGemmF16 path won (the lowering then emits
    // nvteGemmF16, HOMNVGPUToFunc.cpp:125-134)
    return op.kernelName >= 0 && op.splitK >= 1 ? 0 : 1;
  }
  // The manifest object (GemmManifest.h:18-65): size, indexing, the runner's
  // name / activation queries, as GemmProfiler.cu:181-200 walks it.
  using namespace mlir::hands_on_mlir::homnvgpu_kernel;
  int gelu = 0;
  for (size_t i = 0; i < manifest.size(); i++) {
    auto op = manifest[int(i)];
    if (!op.isF16() || manifest.find(op.getName()) != int32_t(i))
      return 2;
    if (op.contains("gelu") != (op.getActivation() == 1))
      return 3;
    gelu += op.getActivation();
  }
  if (gelu == 0 || manifest.getKernel(0).getName() == nullptr)
    return 4;
  printf("%d\n", int(manifest.size()));
  return 0;
}
