#include "common.h"

#include <cstring>
#include <mutex>
#include <vector>

namespace hom {

namespace {
int g_errorMode = 0;
std::string g_lastError;
std::string g_returnedError;
hipStream_t g_stream = nullptr;

struct ScratchBuf {
  void *ptr = nullptr;
  size_t bytes = 0;
};
// One set of slots per stream that has asked for scratch: what is in flight on
// two streams at once must not share partial results.
struct StreamScratch {
  hipStream_t stream = nullptr;
  bool inUse = true;
  ScratchBuf slot[kNumSlots];
};
std::vector<StreamScratch> g_scratch;
std::vector<void *> g_retired; // replaced scratch buffers, kept allocated
int g_scratchGeneration = 0;
} // namespace

int errorMode() { return g_errorMode; }
void setErrorMode(int mode) { g_errorMode = mode; }

void recordError(const char *file, int line, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  const char *base = strrchr(file, '/');
  base = base ? base + 1 : file;
  if (g_errorMode != 2) {
    fprintf(stderr, "hom_amdgpu error: %s (%s:%d)\n", buf, base, line);
    fflush(stderr);
  }
  if (g_errorMode == 0)
    abort();
  g_lastError = buf;
}

const char *takeLastError() {
  g_returnedError.swap(g_lastError);
  g_lastError.clear();
  return g_returnedError.c_str();
}

hipStream_t stream() { return g_stream; }
void setStream(hipStream_t s) { g_stream = s; }

const DeviceInfo &deviceInfo() {
  static DeviceInfo info;
  static bool init = false;
  if (!init) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipGetDeviceProperties(&prop, dev) == hipSuccess) {
      info.computeUnits = prop.multiProcessorCount;
      info.clockKHz = prop.clockRate;
      info.l2Bytes = size_t(prop.l2CacheSize);
    } else {
      info.computeUnits = 256;
      info.clockKHz = 2400000;
    }
    init = true;
  }
  return info;
}

int libraryScratchGeneration() { return g_scratchGeneration; }

void releaseStreamScratch(hipStream_t s) {
  for (StreamScratch &e : g_scratch)
    if (e.inUse && e.stream == s && s != nullptr)
      e.inUse = false;
}

void *libraryScratch(ScratchSlot slot, size_t bytes, bool zero) {
  StreamScratch *mine = nullptr, *spare = nullptr;
  for (StreamScratch &s : g_scratch) {
    if (s.inUse && s.stream == g_stream)
      mine = &s;
    else if (!s.inUse && !spare)
      spare = &s;
  }
  if (!mine) {
    // a set that a finished stream gave back (releaseStreamScratch) serves the
    // next new stream, buffers included
    if (!spare) {
      g_scratch.emplace_back();
      spare = &g_scratch.back();
    }
    mine = spare;
    mine->stream = g_stream;
    mine->inUse = true;
  }
  ScratchBuf &b = mine->slot[slot];
  if (bytes <= b.bytes)
    return b.ptr;
  // Growing never frees the old buffer: queued kernels and captured graphs
  // still hold its address.  It stays allocated (retired) until the process
  // ends; sizes double, so all retired buffers together are smaller than the
  // live one.
  size_t want = 1;
  while (want < bytes)
    want <<= 1;
  void *p = nullptr;
  HOM_HIP_RET(hipMalloc(&p, want), nullptr);
  if (b.ptr) {
    g_retired.push_back(b.ptr);
    g_scratchGeneration++;
  }
  if (zero) {
    HOM_HIP_RET(hipMemset(p, 0, want), nullptr);
  }
  b.ptr = p;
  b.bytes = want;
  return p;
}

namespace {
__global__ void xccOfWorkgroupKernel(unsigned int *out) {
  unsigned int id;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(id));
  if (threadIdx.x == 0)
    out[blockIdx.x] = id & 15u;
}

enum class Placement { kUnknown, kRoundRobin, kOther };
Placement g_placement = Placement::kUnknown;
int g_inKernelMode = 3; // see setSplitKInKernel()
int g_inKernelLaunches = 0;
unsigned int *g_hostWords = nullptr; // [0] misplaced flag, [64..] the probe's output
constexpr int kProbeGroups = 192;
constexpr unsigned kXcds = 8;

// Workgroup i of a launch runs on XCD (first + i) mod 8, whatever XCD the
// launch starts on: checked on a few launches of grids that are not multiples
// of eight (the start then differs from launch to launch).
Placement measurePlacement(hipStream_t s) {
  unsigned int *out = g_hostWords + 64;
  for (int rep = 0; rep < 4; rep++) {
    const int groups = kProbeGroups - rep;
    xccOfWorkgroupKernel<<<dim3(groups), dim3(64), 0, s>>>(out);
    if (hipGetLastError() != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
      return Placement::kOther;
    for (int i = 0; i < groups; i++)
      if (out[i] >= kXcds || out[i] != (out[0] + unsigned(i)) % kXcds)
        return Placement::kOther;
  }
  return Placement::kRoundRobin;
}
} // namespace

void setSplitKInKernel(int mode) {
  g_inKernelMode = mode;
  // Switching (in either direction) forgets a reported violation: the
  // placement is measured again before the form is next used.
  if (g_placement == Placement::kOther)
    g_placement = Placement::kUnknown;
  if (g_hostWords)
    *static_cast<volatile unsigned int *>(g_hostWords) = 0;
}
int splitKInKernelMode() { return g_inKernelMode; }
int splitKInKernelLaunches() { return g_inKernelLaunches; }

bool splitKArrival(hipStream_t s, SplitKArrival *out) {
  if (g_inKernelMode == 0 || g_placement == Placement::kOther)
    return false;
  if (g_placement == Placement::kUnknown) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess ||
        cap != hipStreamCaptureStatusNone)
      return false; // measuring needs a synchronisation
    if (!g_hostWords) {
      void *p = nullptr;
      if (hipHostMalloc(&p, (64 + kProbeGroups) * sizeof(unsigned int),
                        hipHostMallocMapped) != hipSuccess) {
        (void)hipGetLastError();
        g_placement = Placement::kOther;
        return false;
      }
      g_hostWords = static_cast<unsigned int *>(p);
      memset(g_hostWords, 0, (64 + kProbeGroups) * sizeof(unsigned int));
    }
    g_placement = measurePlacement(s);
    if (g_placement != Placement::kRoundRobin)
      return false;
  }
  if (*static_cast<volatile unsigned int *>(g_hostWords) != 0) {
    g_placement = Placement::kOther;
    HOM_CHECK_RET(false, false,
                  "gemm: a split-K launch found the slices of one tile on "
                  "different XCDs and its output may be wrong; later launches "
                  "sum the slices with a second kernel");
  }
  // The words of this stream's set.  Allocating them clears them with a
  // synchronous memset, which a stream under capture must not see: a first use
  // inside a capture sums with the second kernel instead.
  constexpr size_t kWordBytes =
      size_t(kMaxArrivalTiles) * sizeof(unsigned long long);
  void *w = nullptr;
  for (const StreamScratch &e : g_scratch)
    if (e.inUse && e.stream == g_stream && e.slot[kCounters].bytes >= kWordBytes)
      w = e.slot[kCounters].ptr;
  if (!w) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cap) != hipSuccess ||
        cap != hipStreamCaptureStatusNone)
      return false;
    w = libraryScratch(kCounters, kWordBytes, true);
  }
  if (!w)
    return false;
  out->words = static_cast<unsigned long long *>(w);
  out->misplaced = g_hostWords;
  g_inKernelLaunches++;
  return true;
}

} // namespace hom
