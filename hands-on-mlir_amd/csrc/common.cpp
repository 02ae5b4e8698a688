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

} // namespace hom
