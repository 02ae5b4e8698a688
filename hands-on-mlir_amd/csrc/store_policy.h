// Cache policy of the stores that write an operator's result.
//
// The chip is eight XCDs with private, mutually non-coherent L2 caches: what a
// kernel leaves dirty in an L2 is written back when the kernel ends, before
// the next kernel of the stream may start, and that write-back is serial time
// between two dependent launches.  Result stores that carry the system-scope
// bits (sc0 sc1) are written through while the kernel is still computing, so
// the end-of-kernel write-back finds nothing to do.  On the BERT-base encoder
// (88 dependent launches of a few microseconds each) this takes 4 % off a
// forward pass and 0.9 us off the 1024 x 3072 GEMM.  It pays for 16-byte
// stores that together cover whole 64-byte segments; scattered 8-byte stores
// (the attention output, the split-K reduction) and the 4-byte stores of
// outputs whose rows are not 16-byte aligned got slower (1024 x 30522: 77 ->
// 106 us) and keep the default policy.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hom {

// auxiliary (cache policy) operand of the raw buffer store builtins:
// bit 0 = sc0, bit 4 = sc1
constexpr int kWriteThroughAux = 17;

// *p = v with the sc0 sc1 bits.
template <typename V>
__device__ __forceinline__ void storeWriteThrough(V *p, const V &v) {
  static_assert(sizeof(V) == 16 || sizeof(V) == 8 || sizeof(V) == 4 ||
                    sizeof(V) == 2,
                "store width");
  if constexpr (sizeof(V) == 16) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    // The hardware needs two wait states between a store wider than 64
    // bits and a vector instruction that overwrites its data registers.  The
    // compiler inserts them for stores it emits itself but cannot see inside
    // an asm statement, and the registers are dead right after it, so the
    // wait states are part of the statement.
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1"
                 :
                 : "v"(p), "v"(__builtin_bit_cast(u32x4, v))
                 : "memory");
  } else if constexpr (sizeof(V) == 8) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1"
                 :
                 : "v"(p), "v"(__builtin_bit_cast(u32x2, v))
                 : "memory");
  } else if constexpr (sizeof(V) == 4) {
    asm volatile("global_store_dword %0, %1, off sc0 sc1"
                 :
                 : "v"(p), "v"(__builtin_bit_cast(uint32_t, v))
                 : "memory");
  } else {
    asm volatile("global_store_short %0, %1, off sc0 sc1"
                 :
                 : "v"(p), "v"(uint32_t(__builtin_bit_cast(uint16_t, v)))
                 : "memory");
  }
}

// *p = v for 16-byte results of kernels that stream tensors larger than the
// last-level cache (nothing is read again soon): written through and marked
// non-temporal.  A cold in-place read-modify-write stream of 33.5 MB measured
// 4.65 TB/s with default accesses, 5.55 TB/s with the non-temporal hint on
// loads and stores, 5.72 TB/s with this store policy on top (sc1 nt; sc0 sc1
// nt is the same); write-through without the hint 5.49 TB/s.
template <typename V>
__device__ __forceinline__ void storeStreaming(V *p, const V &v) {
  static_assert(sizeof(V) == 16, "store width");
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  // (wait states: see storeWriteThrough)
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1"
               :
               : "v"(p), "v"(__builtin_bit_cast(u32x4, v))
               : "memory");
}

} // namespace hom
