// Shared host-side plumbing for the runtime kernel library: argument checks,
// HIP error handling, the library stream, memref views and grow-only device
// scratch.  Plays the role of include/NVGPUKernels/Utils.h:45-52,179-238 in
// the reference (checkCudaErrors, getDummyPointer, getMulitProcessorCount).
#pragma once

#include "hom_memref.h"
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <string>

namespace hom {

// ---------------------------------------------------------------- errors --
// mode 0: print + abort (reference behaviour); mode 1: print, remember, and
// let the entry point return early; mode 2 (library-internal, used while the
// autotuner probes whether a kernel accepts a problem): remember silently.
int errorMode();
void setErrorMode(int mode);
void recordError(const char *file, int line, const char *fmt, ...)
    __attribute__((format(printf, 3, 4)));
const char *takeLastError();

// Check an argument condition inside a void entry point / runner.  On failure
// either aborts or returns `ret` from the enclosing function.
#define HOM_CHECK_RET(cond, ret, ...)                                          \
  do {                                                                         \
    if (!(cond)) {                                                             \
      ::hom::recordError(__FILE__, __LINE__, __VA_ARGS__);                     \
      return ret;                                                              \
    }                                                                          \
  } while (0)

#define HOM_HIP_RET(expr, ret)                                                 \
  do {                                                                         \
    hipError_t _e = (expr);                                                    \
    if (_e != hipSuccess) {                                                    \
      ::hom::recordError(__FILE__, __LINE__, "HIP error %d (%s) from %s",      \
                         int(_e), hipGetErrorString(_e), #expr);               \
      return ret;                                                              \
    }                                                                          \
  } while (0)

enum class Status : int { kSuccess = 0, kInvalidArgument = 1, kInternal = 2 };

// ---------------------------------------------------------------- stream --
hipStream_t stream();
void setStream(hipStream_t s);

// ------------------------------------------------------------ memref view --
// Equivalent of convertToDynamicMemRefType (HandsOnRunnerUtils.h:37-42): reads
// `data`, `sizes`, `strides`; `offset` is ignored exactly as the reference's
// runners ignore it (e.g. GemmRunner.h:279-284 passes A.data directly).
template <typename T> struct View {
  int64_t rank = 0;
  T *data = nullptr;
  const int64_t *sizes = nullptr;
  const int64_t *strides = nullptr;

  View() = default;
  View(int64_t rank_, void *descriptor) : rank(rank_) {
    if (descriptor) {
      data = static_cast<T *>(static_cast<HomMemRefHeader *>(descriptor)->data);
      sizes = hom_memref_sizes(descriptor);
      strides = hom_memref_strides(descriptor, rank_);
    }
  }
  int64_t numel() const {
    int64_t n = 1;
    for (int64_t i = 0; i < rank; i++)
      n *= sizes[i];
    return n;
  }
  bool contiguous() const {
    int64_t expect = 1;
    for (int64_t i = rank - 1; i >= 0; i--) {
      if (sizes[i] != 1 && strides[i] != expect)
        return false;
      expect *= sizes[i];
    }
    return true;
  }
};

// ---------------------------------------------------------------- device --
struct DeviceInfo {
  int computeUnits = 0;
  int clockKHz = 0;
  size_t l2Bytes = 0;
};
const DeviceInfo &deviceInfo();

// Grow-only device scratch, one buffer per slot and per stream the library has
// been pointed at (setStream): calls in flight on different streams do not
// share partial results.  Slot kWorkspace holds split-K partial tiles, kTemp
// the temporaries of the layer-norm GEMM pair.
// A buffer that has been handed out is never freed while the process lives:
// kernels already enqueued, and HIP graphs captured earlier, keep its address
// in their arguments.  When a slot must grow, a new buffer of at least twice
// the size is allocated and the old one is retired (kept, unused by later
// calls), so retired buffers add up to less than the live one.
enum ScratchSlot { kWorkspace = 0, kCounters = 1, kTemp = 2, kNumSlots = 3 };
// Returns nullptr (after recording an error) on allocation failure.  `zero`
// clears newly allocated memory once, at allocation time.
void *libraryScratch(ScratchSlot slot, size_t bytes, bool zero);
// Number of times any slot has been replaced by a larger buffer (tests).
int libraryScratchGeneration();
// The caller is done with stream `s` (everything enqueued on it has finished
// and no graph captured on it will be replayed): its buffers go to the next
// stream that asks.  Without this call they stay with `s` until the process
// ends.  The null stream's set is never given away.
void releaseStreamScratch(hipStream_t s);

// In-kernel split-K reduction.  The K slices of a tile add one to the tile's
// arrival word (slot kCounters, zero between launches: the slice that arrives
// last sums the partial tiles and puts the word back to zero).  That slice
// reads the others' partial tiles through its own L2, so the form is only
// right when all slices of a tile run on one XCD; the launcher arranges that
// from the round-robin placement of workgroups over the XCDs, which this
// function measures once per process with a tiny kernel before it hands out
// the words.  Returns nullptr -- sum with a second kernel instead -- while
// `s` is being captured before that measurement has run, when the placement
// is not the expected one, when a kernel has reported slices of one tile on
// different XCDs (an error is recorded too), or after setSplitKInKernel(0).
constexpr int kMaxArrivalTiles = 8192;
struct SplitKArrival {
  unsigned long long *words; // [kMaxArrivalTiles]
  unsigned int *misplaced;   // host-visible; kernels set it to 1 on a violation
};
bool splitKArrival(hipStream_t s, SplitKArrival *out);
// mode 0: never; 1: wherever the launch keeps a tile's slices on one XCD;
// 2: like 1, and the launcher skips that condition (slices then land on
// different XCDs and the kernels' check must report it: what the tests of that
// check use); 3 (the default): like 1, but only where it measured faster than
// the second kernel (splitKInKernelPays()).
void setSplitKInKernel(int mode);
int splitKInKernelMode();
// Measured on MI355X over tiles, shapes and split factors: the last arriver
// walks its tile's slices alone, so the form pays with small tiles (a partial
// tile of at most 32 KB), few slices, and a launch that is resident at once
// with room to spare; otherwise the second kernel, which spreads the sum over
// the whole chip, is as fast or faster.
inline bool splitKInKernelPays(int tileElems, int slices, long long tiles) {
  return tileElems <= 128 * 64 && slices <= 6 && tiles * slices <= 512;
}
int splitKInKernelLaunches(); // launches that used the in-kernel form (tests)

} // namespace hom
