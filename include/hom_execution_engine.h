/* Host-side loader for modules compiled by hands-on-opt: the role of
 * mlir::hands_on_mlir::ExecutionEngine in the reference
 * (include/ExecutionEngine/ExecutionEngine.h:27-171,
 * lib/ExecutionEngine/ExecutionEngine.cpp:22-97), without the LLVM support
 * types in its interface.
 *
 * A compiled module is a shared object that, for every public function <f>,
 * exports four symbols with the packed calling convention `void (*)(void **)`
 * (lib/Conversions/Function/UnifyLLVMFuncInterface.cpp:60-131: slot i of the
 * array points to argument i, the slot after the last argument points to where
 * the result is stored; an unranked memref argument takes two slots, its rank
 * (int64_t) and its descriptor pointer):
 *   _hom_ciface_<f>_argNum    -> int32_t: number of tensors the module manages
 *   _hom_ciface_<f>_initFn    -> that many {int64_t rank; void *descriptor}
 *                                (weights via allocConstantNVGPU*, intermediates
 *                                via alloc*MemRefNVGPU*; hoisted out of <f> by
 *                                lib/Conversions/Function/ExtractInitFunc.cpp:60-276)
 *   _hom_ciface_<f>           (managed tensors..., user arguments...) -> result
 *   _hom_ciface_<f>_deallocFn (managed tensors...)
 * The module itself links against libhom_amdgpu_runner_utils.so for the
 * operator entry points (hom_amdgpu_runner_utils.h).
 */
#ifndef HOM_EXECUTION_ENGINE_H_
#define HOM_EXECUTION_ENGINE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct HomEngine HomEngine;

/* dlopen()s the module (ExecutionEngine::ExecutionEngine, ExecutionEngine.h:31-36).
 * Returns NULL when the file cannot be loaded; homEngineLastError(NULL) says why. */
HomEngine *homEngineOpen(const char *sharedObjectPath);

/* _hom_ciface_<func>_argNum (ExecutionEngine::invokeInit, ExecutionEngine.cpp:74-83).
 * Returns -1 when the symbol is missing. */
int32_t homEngineArgNum(HomEngine *engine, const char *func);

/* ExecutionEngine::invoke (ExecutionEngine.h:118-135): on the first call for
 * <func> runs _argNum and _initFn and keeps the managed tensors; then calls
 * _hom_ciface_<func> with the managed tensors (two slots each) followed by the
 * caller's `numSlots` slots -- pointers to the argument values in declaration
 * order, a pointer to the result storage last when the function returns a value.
 * Returns 0, or -1 with homEngineLastError() set. */
int homEngineInvoke(HomEngine *engine, const char *func, void **slots, int32_t numSlots);

/* Calls _hom_ciface_<func>_deallocFn on the managed tensors of <func> (device
 * buffers) and forgets them.  The reference never calls its dealloc function;
 * its destructor only frees the descriptors. */
int homEngineDealloc(HomEngine *engine, const char *func);

/* ExecutionEngine::~ExecutionEngine (ExecutionEngine.h:38-46): frees the host
 * descriptors of the managed tensors still held and closes the module. */
void homEngineClose(HomEngine *engine);

/* Message of the last failure on this engine (engine == NULL: of the last
 * failed homEngineOpen on this thread).  Never NULL. */
const char *homEngineLastError(HomEngine *engine);

#ifdef __cplusplus
}
#endif
#endif /* HOM_EXECUTION_ENGINE_H_ */
