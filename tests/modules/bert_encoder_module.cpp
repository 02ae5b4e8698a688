// Stand-in for a module compiled by hands-on-opt: a post-LN BERT encoder with
// static shapes, written by hand in the form the compiler's last passes leave
// (lib/Conversions/Function/HOMNVGPUToFunc.cpp: operator calls and their
// operand order; ExtractInitFunc.cpp:60-276: weights and intermediates hoisted
// into <f>_initFn and prepended to <f>'s arguments, <f>_argNum, <f>_deallocFn;
// UnifyLLVMFuncInterface.cpp:60-131: every function behind a
// `_hom_ciface_<f>(void **)` wrapper that loads argument i through slot i and
// stores the result through the slot after the last argument).  The compiler
// cannot run where these tests run, so the tests build this file instead and
// load it through the execution engine: it exercises the same symbols, calling
// convention and ownership rules a real module does.
//
// Shapes are compile-time constants, as in generated code:
//   -DHOM_LAYERS= -DHOM_HIDDEN= -DHOM_HEADS= -DHOM_FFN= -DHOM_BATCH= -DHOM_SEQ= -DHOM_VOCAB=
// Constants (allocConstantNVGPUF16(idx), files in $HOM_CONSTANT_DIR):
//   0 word embeddings [1, V, H]; 1 position+type embeddings [1, S, H];
//   2 + 4l .. 5 + 4l: Wqkv [1, H, 3H], Wo [1, H, H], W1 [1, H, F], W2 [1, F, H] of layer l;
//   with -DHOM_LM_HEAD (the masked-LM head of BertForMaskedLM, the graph the
//   reference's examples/torch/bert/bert.cu runs to logits [b, s, vocab]):
//   2 + 4L transform dense [1, H, H], 3 + 4L decoder [1, H, V]; forward then
//   returns the logits instead of the hidden states.
// -DHOM_GEMM_NUM=n selects a manifest kernel the way the autotune pass bakes one
// in (0: the library chooses); -DHOM_USE_NVTE routes GEMMs to nvteGemmF16 with
// [1, N, K] weights instead.
#include "hom_amdgpu_runner_utils.h"

#include <cmath>
#include <cstdlib>
#include <cstring>

namespace {
constexpr int L = HOM_LAYERS, H = HOM_HIDDEN, HEADS = HOM_HEADS, F = HOM_FFN;
constexpr int B = HOM_BATCH, S = HOM_SEQ, V = HOM_VOCAB;
#ifndef HOM_GEMM_NUM
#define HOM_GEMM_NUM 0
#endif
#ifdef HOM_LM_HEAD
constexpr int kHead = 1;
#else
constexpr int kHead = 0;
#endif
constexpr int kConstants = 2 + 4 * L + 2 * kHead;
// + cu, emb, h, qkv, attn, ffn (+ transform output, logits)
constexpr int kManaged = kConstants + 6 + 2 * kHead;

typedef C_UnrankedMemRefType M;

void gemm(const M &a, const M &w, const M &d, int64_t act, float beta) {
#ifdef HOM_USE_NVTE
  nvteGemmF16(a.rank, a.descriptor, false, w.rank, w.descriptor, true, d.rank,
              d.descriptor, d.rank, d.descriptor, act, 1.0f, beta, 0, 0);
#else
  cutlassGemmF16(a.rank, a.descriptor, false, w.rank, w.descriptor, false,
                 d.rank, d.descriptor, d.rank, d.descriptor, act, 1.0f, beta,
                 HOM_GEMM_NUM, 1);
#endif
}

// forward(managed tensors..., input_ids, attention_mask) -> hidden states
M forward(const M *t, M ids, M mask) {
  const M &word = t[0], &posType = t[1];
  const M &cu = t[kConstants], &emb = t[kConstants + 1], &h = t[kConstants + 2];
  const M &qkv = t[kConstants + 3], &attn = t[kConstants + 4], &ffn = t[kConstants + 5];
  thrustCuSeqLenI64(mask.rank, mask.descriptor, cu.rank, cu.descriptor);
  thrustGatherF16(ids.rank, ids.descriptor, word.rank, word.descriptor, emb.rank,
                  emb.descriptor);
  thrustElementwiseAddF16(emb.rank, emb.descriptor, posType.rank,
                          posType.descriptor, h.rank, h.descriptor);
  nvteLayernormF16(h.rank, h.descriptor, 1e-12f);
  const float scale = 1.0f / std::sqrt(float(H / HEADS));
  for (int l = 0; l < L; l++) {
    const M *w = t + 2 + 4 * l;
    gemm(h, w[0], qkv, 0, 0.0f);
    nvteBertAttentionF16(qkv.rank, qkv.descriptor, cu.rank, cu.descriptor,
                         attn.rank, attn.descriptor, scale, HEADS);
    gemm(attn, w[1], h, 0, 1.0f); // residual: C aliases D
    nvteLayernormF16(h.rank, h.descriptor, 1e-12f);
    gemm(h, w[2], ffn, 1, 0.0f);  // activation 1: GELU
    gemm(ffn, w[3], h, 0, 1.0f);
    nvteLayernormF16(h.rank, h.descriptor, 1e-12f);
  }
  const M *result = &h;
  if (kHead) {
    const M &wt = t[2 + 4 * L], &wd = t[3 + 4 * L];
    const M &tr = t[kConstants + 6], &logits = t[kConstants + 7];
    gemm(h, wt, tr, 1, 0.0f);
    nvteLayernormF16(tr.rank, tr.descriptor, 1e-12f);
    gemm(tr, wd, logits, 0, 0.0f);
    result = &logits;
  }
  // A returned unranked memref carries a descriptor the caller frees.
  const size_t bytes = sizeof(int64_t) * (3 + 2 * 3);
  M out{result->rank, std::malloc(bytes)};
  std::memcpy(out.descriptor, result->descriptor, bytes);
  return out;
}
} // namespace

extern "C" {
__attribute__((visibility("default"))) void _hom_ciface_forward_argNum(void **slots) {
  *static_cast<int32_t *>(slots[0]) = kManaged;
}

__attribute__((visibility("default"))) void _hom_ciface_forward_initFn(void **slots) {
  M *out = static_cast<M *>(slots[0]); // kManaged consecutive {rank, descriptor}
  for (int i = 0; i < kConstants; i++)
    out[i] = allocConstantNVGPUF16(i);
  out[kConstants] = alloc1DMemRefNVGPUI32(B + 1);
  out[kConstants + 1] = alloc3DMemRefNVGPUF16(B, S, H);
  out[kConstants + 2] = alloc3DMemRefNVGPUF16(B, S, H);
  out[kConstants + 3] = alloc3DMemRefNVGPUF16(B, S, 3 * H);
  out[kConstants + 4] = alloc3DMemRefNVGPUF16(B, S, H);
  out[kConstants + 5] = alloc3DMemRefNVGPUF16(B, S, F);
  if (kHead) {
    out[kConstants + 6] = alloc3DMemRefNVGPUF16(B, S, H);
    out[kConstants + 7] = alloc3DMemRefNVGPUF16(B, S, V);
  }
}

__attribute__((visibility("default"))) void _hom_ciface_forward(void **slots) {
  M t[kManaged];
  for (int i = 0; i < kManaged; i++) {
    t[i].rank = *static_cast<int64_t *>(slots[2 * i]);
    t[i].descriptor = *static_cast<void **>(slots[2 * i + 1]);
  }
  void **user = slots + 2 * kManaged;
  M ids{*static_cast<int64_t *>(user[0]), *static_cast<void **>(user[1])};
  M mask{*static_cast<int64_t *>(user[2]), *static_cast<void **>(user[3])};
  *static_cast<M *>(user[4]) = forward(t, ids, mask);
}

__attribute__((visibility("default"))) void _hom_ciface_forward_deallocFn(void **slots) {
  for (int i = 0; i < kManaged; i++) {
    const int64_t rank = *static_cast<int64_t *>(slots[2 * i]);
    void *desc = *static_cast<void **>(slots[2 * i + 1]);
    if (i == kConstants)
      deallocNVGPUI32(rank, desc);
    else
      deallocNVGPUF16(rank, desc);
  }
}
}
