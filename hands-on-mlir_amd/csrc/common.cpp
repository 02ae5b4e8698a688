#include "common.h"

#include <cstring>
#include <mutex>

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
ScratchBuf g_scratch[kNumSlots];
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
  fprintf(stderr, "hom_amdgpu error: %s (%s:%d)\n", buf, base, line);
  fflush(stderr);
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

void *scratch(ScratchSlot slot, size_t bytes, bool zero) {
  ScratchBuf &b = g_scratch[slot];
  if (bytes <= b.bytes)
    return b.ptr;
  // Growing replaces the buffer: wait for queued work that may still use the
  // old one.  Sizes are rounded up generously so this is rare.
  size_t want = 1;
  while (want < bytes)
    want <<= 1;
  if (b.ptr) {
    HOM_HIP_RET(hipDeviceSynchronize(), nullptr);
    HOM_HIP_RET(hipFree(b.ptr), nullptr);
    b.ptr = nullptr;
    b.bytes = 0;
  }
  void *p = nullptr;
  HOM_HIP_RET(hipMalloc(&p, want), nullptr);
  if (zero) {
    HOM_HIP_RET(hipMemset(p, 0, want), nullptr);
  }
  b.ptr = p;
  b.bytes = want;
  return p;
}

} // namespace hom
