// Loader for hands-on-opt compiled modules: dlopen + the packed calling
// convention, see include/hom_execution_engine.h.  Host only: nothing here
// touches the GPU; the module's own code calls the operator library.
#include "hom_execution_engine.h"
#include "hom_memref.h"

#include <cstdlib>
#include <dlfcn.h>
#include <string>
#include <unordered_map>
#include <vector>

#define ENGINE_EXPORT extern "C" __attribute__((visibility("default")))

struct HomEngine {
  void *handle = nullptr;
  std::string error;
  // tensors the module manages, per public function (weights, intermediates)
  std::unordered_map<std::string, std::vector<C_UnrankedMemRefType>> managed;
};

namespace {
thread_local std::string openError;
using PackedFn = void (*)(void **);

PackedFn lookup(HomEngine *e, const std::string &func) {
  const std::string name = "_hom_ciface_" + func;
  dlerror();
  void *sym = dlsym(e->handle, name.c_str());
  const char *err = dlerror();
  if (err || !sym) {
    e->error = err ? err : ("symbol " + name + " is null");
    return nullptr;
  }
  return reinterpret_cast<PackedFn>(sym);
}

// Runs _argNum and _initFn once per function.  _initFn returns its tensors as
// one struct of {rank, descriptor} pairs, stored where the slot after its (zero)
// arguments points: a contiguous array of C_UnrankedMemRefType.
std::vector<C_UnrankedMemRefType> *ensureInit(HomEngine *e, const std::string &func) {
  auto it = e->managed.find(func);
  if (it != e->managed.end())
    return &it->second;
  PackedFn argNum = lookup(e, func + "_argNum");
  PackedFn init = lookup(e, func + "_initFn");
  if (!argNum || !init)
    return nullptr;
  int32_t n = 0;
  void *numSlots[1] = {&n};
  argNum(numSlots);
  if (n < 0) {
    e->error = "module reports a negative number of managed tensors";
    return nullptr;
  }
  std::vector<C_UnrankedMemRefType> tensors(size_t(n), C_UnrankedMemRefType{0, nullptr});
  // the reference passes one slot per field of every tensor; only the first is
  // read (it is where the whole result struct goes)
  std::vector<void *> slots;
  for (auto &t : tensors) {
    slots.push_back(&t.rank);
    slots.push_back(&t.descriptor);
  }
  if (slots.empty())
    slots.push_back(nullptr);
  init(slots.data());
  return &e->managed.emplace(func, std::move(tensors)).first->second;
}
} // namespace

ENGINE_EXPORT HomEngine *homEngineOpen(const char *path) {
  void *h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!h) {
    const char *err = dlerror();
    openError = err ? err : "dlopen failed";
    return nullptr;
  }
  auto *e = new HomEngine();
  e->handle = h;
  return e;
}

ENGINE_EXPORT int32_t homEngineArgNum(HomEngine *e, const char *func) {
  PackedFn argNum = lookup(e, std::string(func) + "_argNum");
  if (!argNum)
    return -1;
  int32_t n = 0;
  void *slots[1] = {&n};
  argNum(slots);
  return n;
}

ENGINE_EXPORT int homEngineInvoke(HomEngine *e, const char *func, void **user,
                                  int32_t numSlots) {
  std::vector<C_UnrankedMemRefType> *tensors = ensureInit(e, func);
  PackedFn fn = tensors ? lookup(e, func) : nullptr;
  if (!fn)
    return -1;
  std::vector<void *> slots;
  slots.reserve(tensors->size() * 2 + size_t(numSlots));
  for (auto &t : *tensors) {
    slots.push_back(&t.rank);
    slots.push_back(&t.descriptor);
  }
  for (int32_t i = 0; i < numSlots; i++)
    slots.push_back(user[i]);
  fn(slots.data());
  return 0;
}

ENGINE_EXPORT int homEngineDealloc(HomEngine *e, const char *func) {
  auto it = e->managed.find(func);
  if (it == e->managed.end())
    return 0;
  PackedFn fn = lookup(e, std::string(func) + "_deallocFn");
  if (!fn)
    return -1;
  std::vector<void *> slots;
  for (auto &t : it->second) {
    slots.push_back(&t.rank);
    slots.push_back(&t.descriptor);
  }
  slots.push_back(nullptr);
  fn(slots.data());
  // deallocNVGPU* released the device buffers; the descriptors are ours
  for (auto &t : it->second)
    free(t.descriptor);
  e->managed.erase(it);
  return 0;
}

ENGINE_EXPORT void homEngineClose(HomEngine *e) {
  if (!e)
    return;
  for (auto &kv : e->managed)
    for (auto &t : kv.second)
      free(t.descriptor);
  if (e->handle)
    dlclose(e->handle);
  delete e;
}

ENGINE_EXPORT const char *homEngineLastError(HomEngine *e) {
  return e ? e->error.c_str() : openError.c_str();
}
