// Host driver for a lowered BERT encoder: the stand-in for the code that
// hands-on-opt generates (`_hom_ciface_forward` plus its `_initFn`) and for the
// reference's ExecutionEngine (lib/ExecutionEngine/ExecutionEngine.cpp:73-97,
// examples/torch/bert/bert.cu:81-127).
//
// init:    every weight and every intermediate is allocated ONCE through the
//          library's alloc* entry points (what ExtractInitFunc hoists,
//          lib/Conversions/Function/ExtractInitFunc.cpp:94-188);
// forward: a straight-line list of C-ABI calls, no host control flow and no
//          synchronisation -- the list in HOMNVGPUToFunc.cpp for
//            cu_seqlens; gather + add + layernorm (embeddings);
//            per layer: QKV GEMM, attention, out-proj GEMM (+residual, in
//            place), layernorm, FFN1 GEMM+GELU, FFN2 GEMM (+residual, in
//            place), layernorm;
//            optionally the masked-LM head of the reference's BertForMaskedLM
//            graph (examples/torch/bert/bert.cu:25,140-163: logits
//            [b, s, vocab]): dense + GELU, layernorm, vocabulary projection.
// Because that list is static, the driver can also capture it once into a HIP
// graph and replay it, which removes the per-call launch overhead that
// dominates at batch 8 x seq 128.
//
// Everything goes through the extern "C" boundary; nothing here reaches into
// the library's internals.
#include "hom_amdgpu_runner_utils.h"

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define DRV_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

struct Tensor {
  C_UnrankedMemRefType m{0, nullptr};
  void *data() const { return m.descriptor ? hom_memref_data(m.descriptor) : nullptr; }
  void release() {
    if (m.descriptor) {
      deallocNVGPUF16(m.rank, m.descriptor);
      free(m.descriptor);
      m.descriptor = nullptr;
    }
  }
};

struct LayerWeights {
  Tensor wqkv, wo, w1, w2; // [1,K,N] (manifest path) or [1,N,K] (nvte path)
};

// How one GEMM role of the graph is called.  nk: the weight is stored as
// [1, N, K] and the call goes to nvteGemmF16 -- what the reference's compiler
// emits for a matmul whose autotune result was "nvte" (kernel number 0);
// otherwise cutlassGemmF16 with the manifest kernel gemmNum.
struct GemmChoice {
  int32_t gemmNum = 0; // 1-based manifest index, 0 = library picks
  int32_t splitK = 1;
  bool nk = false;
};

} // namespace

struct HomBertEncoder {
  int layers, hidden, heads, ffn, batch, seq, vocab;
  int gemmMode; // 0 = nvteGemmF16 (B pre-transposed), 1 = cutlassGemmF16 +
                // tuned table / heuristic, 2 = cutlassGemmF16 + live autotune
  int geluForm; // 0 erf, 1 tanh (manifest path only; nvte path is tanh)
  float eps;
  std::vector<LayerWeights> w;
  Tensor wordEmb;   // [1, vocab, H]
  Tensor posType;   // [1, seq, H]  (position + token-type rows, constant folded)
  Tensor ids;       // int64 [b, s]   (descriptor built by hand, see create)
  Tensor mask;      // int64 [b, s]
  Tensor cu;        // int32 [b+1]
  Tensor h, emb, qkv, attn, f;
  // masked-LM head (homBertEnableLmHead): transform weight [1,H,H], decoder
  // weight [1,H,V] ([1,H,H] / [1,V,H] on the nvte path), transform output and
  // logits
  int32_t roleLayout[6] = {-1, -1, -1, -1, -1, -1};
  bool lmHead = false;
  Tensor wTransform, wDecoder, t, logits;
  GemmChoice cQkv, cOut, cFfn1, cFfn2, cTransform, cDecoder;
  // Folded layer norms (homBertFoldLayernorm): the column sums of every Wqkv
  // and W1 (fp32, device), two buffers of partial row sums that the
  // residual GEMMs write alternately, and the number of pieces in them.
  bool foldLn = false;
  std::vector<float *> colSumQkv, colSumW1;
  float *rowSums[2] = {nullptr, nullptr};
  int32_t foldPieces = 0;
  hipStream_t stream = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t graphExec = nullptr;
  hipEvent_t evStart = nullptr, evStop = nullptr;
};

namespace {

bool hipOk(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    fprintf(stderr, "hom_bert_driver: %s failed: %s\n", what,
            hipGetErrorString(e));
    return false;
  }
  return true;
}

// int64 [b, s] tensor: there is no alloc entry point for it in the boundary
// (the reference's driver builds these with allocHelper itself, bert.cu:27-78).
Tensor allocI64_2D(int64_t a, int64_t b) {
  Tensor t;
  auto *d = static_cast<HomStridedMemRef2 *>(malloc(sizeof(HomStridedMemRef2)));
  void *dev = nullptr;
  if (!hipOk(hipMalloc(&dev, size_t(a) * b * sizeof(int64_t)), "hipMalloc")) {
    free(d);
    return t;
  }
  d->basePtr = d->data = dev;
  d->offset = 0;
  d->sizes[0] = a;
  d->sizes[1] = b;
  d->strides[0] = b;
  d->strides[1] = 1;
  t.m.rank = 2;
  t.m.descriptor = d;
  return t;
}

void gemm(HomBertEncoder *e, const Tensor &a, const Tensor &w, const Tensor &c,
          const Tensor &d, int64_t act, float beta, const GemmChoice &ch) {
  (void)e;
  if (ch.nk) {
    nvteGemmF16(a.m.rank, a.m.descriptor, false, w.m.rank, w.m.descriptor, true,
                c.m.rank, c.m.descriptor, d.m.rank, d.m.descriptor, act, 1.0f,
                beta, 0, 1);
  } else {
    cutlassGemmF16(a.m.rank, a.m.descriptor, false, w.m.rank, w.m.descriptor,
                   false, c.m.rank, c.m.descriptor, d.m.rank, d.m.descriptor,
                   act, 1.0f, beta, ch.gemmNum, ch.splitK);
  }
}

// layout: 0 row-major weight, 1 [N, K] weight, -1 decide here (gemmMode 0: always
// [N, K]; 1: what the shipped table prefers; 2: what the live autotuner finds).
// nvteGemmF16 computes the tanh form of GELU only, so a GELU role of an erf
// graph stays on the manifest path; pinning such a role to [N, K] is refused
// (returns false) instead of silently computing the other GELU.
bool chooseGemm(HomBertEncoder *e, int64_t M, int64_t N, int64_t K, int64_t act,
                float beta, int layout, GemmChoice *out) {
  const bool nkAllowed = act == 0 || e->geluForm == 1 || e->gemmMode == 0;
  int64_t idx = -1;
  int32_t sk = 1;
  out->nk = false;
  if (layout == 1 && !nkAllowed) {
    fprintf(stderr, "hom_bert_driver: a GELU role of an erf-GELU graph cannot "
                    "take [N, K] weights: nvteGemmF16 computes the tanh form\n");
    return false;
  }
  if (e->gemmMode == 0 || layout == 1) {
    out->nk = true;
  } else if (e->gemmMode == 2) {
    homGemmProfile(M, N, K, act, 1.0f, beta, &idx, &sk, nullptr);
    if (idx < 0 && layout == -1 && nkAllowed)
      out->nk = true;
    else if (idx < 0)
      homGemmProfileLayout(M, N, K, act, 1.0f, beta, 0, &idx, &sk, nullptr);
  } else {
    if (layout == -1 && nkAllowed && homGemmPrefersNvte(M, N, K, act))
      out->nk = true;
    else
      homGemmSelect(M, N, K, act, &idx, &sk);
  }
  out->gemmNum = out->nk ? 0 : int32_t(idx + 1);
  out->splitK = out->nk ? 1 : sk;
  return true;
}

void callList(HomBertEncoder *e, int fromIds) {
  thrustCuSeqLenI64(e->mask.m.rank, e->mask.m.descriptor, e->cu.m.rank,
                    e->cu.m.descriptor);
  if (fromIds) {
    thrustGatherF16(e->ids.m.rank, e->ids.m.descriptor, e->wordEmb.m.rank,
                    e->wordEmb.m.descriptor, e->emb.m.rank,
                    e->emb.m.descriptor);
    thrustElementwiseAddF16(e->emb.m.rank, e->emb.m.descriptor,
                            e->posType.m.rank, e->posType.m.descriptor,
                            e->h.m.rank, e->h.m.descriptor);
    nvteLayernormF16(e->h.m.rank, e->h.m.descriptor, e->eps);
  }
  const float scale = 1.0f / sqrtf(float(e->hidden / e->heads));
  const int64_t geluAct = e->gemmMode == 0 ? 1 : (e->geluForm == 1 ? 2 : 1);
  if (e->foldLn) {
    // The same graph with the two layer norms of every layer folded into the
    // GEMMs around them: the residual GEMMs (out-projection, FFN2) leave the
    // un-normalised sum in h together with the partial row sums of it, and
    // whoever reads h next -- the following GEMM as its A operand, the next
    // residual GEMM as its source -- normalises on the fly.  One real layer
    // norm remains, behind the last layer.  5 launches per layer instead of 7.
    auto folded = [&](const Tensor &a, const Tensor &w, const Tensor &c,
                      const Tensor &d, int32_t mode, int64_t act, float beta,
                      const float *statsIn, const float *colSum,
                      float *statsOut) {
      homGemmFoldedLayernormF16(a.m.rank, a.m.descriptor, w.m.rank,
                                w.m.descriptor, c.m.rank, c.m.descriptor,
                                d.m.rank, d.m.descriptor, mode, act, 1.0f, beta,
                                statsIn, e->foldPieces, e->eps, colSum,
                                statsOut, 0);
    };
    const float *stats = nullptr; // h is normalised (embeddings) at the start
    for (int l = 0; l < e->layers; l++) {
      const LayerWeights &w = e->w[size_t(l)];
      folded(e->h, w.wqkv, e->qkv, e->qkv, 1, 0, 0.0f, stats,
             e->colSumQkv[size_t(l)], nullptr);
      nvteBertAttentionF16(e->qkv.m.rank, e->qkv.m.descriptor, e->cu.m.rank,
                           e->cu.m.descriptor, e->attn.m.rank,
                           e->attn.m.descriptor, scale, e->heads);
      folded(e->attn, w.wo, e->h, e->h, 2, 0, 1.0f, stats, nullptr,
             e->rowSums[0]);
      folded(e->h, w.w1, e->f, e->f, 1, 1, 0.0f, e->rowSums[0],
             e->colSumW1[size_t(l)], nullptr);
      folded(e->f, w.w2, e->h, e->h, 2, 0, 1.0f, e->rowSums[0], nullptr,
             e->rowSums[1]);
      stats = e->rowSums[1];
    }
    nvteLayernormF16(e->h.m.rank, e->h.m.descriptor, e->eps);
  } else
  for (int l = 0; l < e->layers; l++) {
    const LayerWeights &w = e->w[l];
    gemm(e, e->h, w.wqkv, e->qkv, e->qkv, 0, 0.0f, e->cQkv);
    nvteBertAttentionF16(e->qkv.m.rank, e->qkv.m.descriptor, e->cu.m.rank,
                         e->cu.m.descriptor, e->attn.m.rank,
                         e->attn.m.descriptor, scale, e->heads);
    gemm(e, e->attn, w.wo, e->h, e->h, 0, 1.0f, e->cOut);
    nvteLayernormF16(e->h.m.rank, e->h.m.descriptor, e->eps);
    gemm(e, e->h, w.w1, e->f, e->f, geluAct, 0.0f, e->cFfn1);
    gemm(e, e->f, w.w2, e->h, e->h, 0, 1.0f, e->cFfn2);
    nvteLayernormF16(e->h.m.rank, e->h.m.descriptor, e->eps);
  }
  if (e->lmHead) {
    // BertLMPredictionHead with default-initialised (folded away) biases and
    // affine parameters: t = LN(GELU(h Wt)); logits = t Wd
    gemm(e, e->h, e->wTransform, e->t, e->t, geluAct, 0.0f, e->cTransform);
    nvteLayernormF16(e->t.m.rank, e->t.m.descriptor, e->eps);
    gemm(e, e->t, e->wDecoder, e->logits, e->logits, 0, 0.0f, e->cDecoder);
  }
}

} // namespace

// gemmMode / geluForm as documented on HomBertEncoder.  roleLayout: weight
// layout per GEMM role (QKV, out-proj, FFN1, FFN2, LM transform, LM decoder):
// 0 [K, N] + cutlassGemmF16, 1 [N, K] + nvteGemmF16, -1 (or a null pointer) the
// driver decides, see chooseGemm.
DRV_EXPORT HomBertEncoder *
homBertCreateWithLayout(int layers, int hidden, int heads, int ffn, int batch,
                        int seq, int vocab, int gemmMode, int geluForm,
                        const int32_t *roleLayout) {
  auto *e = new HomBertEncoder();
  e->layers = layers;
  e->hidden = hidden;
  e->heads = heads;
  e->ffn = ffn;
  e->batch = batch;
  e->seq = seq;
  e->vocab = vocab;
  e->gemmMode = gemmMode;
  e->geluForm = geluForm;
  e->eps = 1e-12f;
  e->w.resize(size_t(layers));
  for (int r = 0; r < 6; r++)
    e->roleLayout[r] = roleLayout ? roleLayout[r] : -1;
  {
    const int64_t M = int64_t(batch) * seq;
    const int64_t gelu = geluForm == 1 ? 2 : 1;
    // the LM transform is a GELU role too; its layout is checked here so that
    // a bad pin fails at creation, not at homBertEnableLmHead
    const bool transformOk =
        !(e->roleLayout[4] == 1 && geluForm == 0 && gemmMode != 0);
    if (!chooseGemm(e, M, 3 * hidden, hidden, 0, 0.0f, e->roleLayout[0], &e->cQkv) ||
        !chooseGemm(e, M, hidden, hidden, 0, 1.0f, e->roleLayout[1], &e->cOut) ||
        !chooseGemm(e, M, ffn, hidden, gelu, 0.0f, e->roleLayout[2], &e->cFfn1) ||
        !chooseGemm(e, M, hidden, ffn, 0, 1.0f, e->roleLayout[3], &e->cFfn2) ||
        !transformOk) {
      if (!transformOk)
        fprintf(stderr, "hom_bert_driver: the LM transform of an erf-GELU graph "
                        "cannot take [N, K] weights\n");
      delete e;
      return nullptr;
    }
  }
  for (auto &w : e->w) {
    w.wqkv.m = e->cQkv.nk ? alloc3DMemRefNVGPUF16(1, 3 * hidden, hidden)
                          : alloc3DMemRefNVGPUF16(1, hidden, 3 * hidden);
    w.wo.m = alloc3DMemRefNVGPUF16(1, hidden, hidden);
    w.w1.m = e->cFfn1.nk ? alloc3DMemRefNVGPUF16(1, ffn, hidden)
                         : alloc3DMemRefNVGPUF16(1, hidden, ffn);
    w.w2.m = e->cFfn2.nk ? alloc3DMemRefNVGPUF16(1, hidden, ffn)
                         : alloc3DMemRefNVGPUF16(1, ffn, hidden);
  }
  e->wordEmb.m = alloc3DMemRefNVGPUF16(1, vocab, hidden);
  e->posType.m = alloc3DMemRefNVGPUF16(1, seq, hidden);
  e->ids = allocI64_2D(batch, seq);
  e->mask = allocI64_2D(batch, seq);
  e->cu.m = alloc1DMemRefNVGPUI32(batch + 1);
  e->h.m = alloc3DMemRefNVGPUF16(batch, seq, hidden);
  e->emb.m = alloc3DMemRefNVGPUF16(batch, seq, hidden);
  e->qkv.m = alloc3DMemRefNVGPUF16(batch, seq, 3 * hidden);
  e->attn.m = alloc3DMemRefNVGPUF16(batch, seq, hidden);
  e->f.m = alloc3DMemRefNVGPUF16(batch, seq, ffn);
  if (!hipOk(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking),
             "hipStreamCreate") ||
      !hipOk(hipEventCreate(&e->evStart), "hipEventCreate") ||
      !hipOk(hipEventCreate(&e->evStop), "hipEventCreate"))
    return e;
  return e;
}

DRV_EXPORT HomBertEncoder *homBertCreate(int layers, int hidden, int heads,
                                         int ffn, int batch, int seq, int vocab,
                                         int gemmMode, int geluForm) {
  return homBertCreateWithLayout(layers, hidden, heads, ffn, batch, seq, vocab,
                                 gemmMode, geluForm, nullptr);
}

// 1 when the weight of a GEMM role (0 QKV, 1 out-proj, 2 FFN1, 3 FFN2, 4 LM
// transform, 5 LM decoder) is stored as [N, K]; uploads must match.
DRV_EXPORT int homBertRoleIsNK(HomBertEncoder *e, int role) {
  const GemmChoice *c[6] = {&e->cQkv,  &e->cOut,       &e->cFfn1,
                            &e->cFfn2, &e->cTransform, &e->cDecoder};
  return role >= 0 && role < 6 && c[role]->nk ? 1 : 0;
}

// Adds the masked-LM head to the call list: allocates its two weights
// (upload with which = 6 transform [H,H], 7 decoder [H,V]; [N,K] layouts when
// gemmMode == 0), the transform buffer and the logits [b, s, vocab].  A graph
// captured before this call must be captured again.
DRV_EXPORT int homBertEnableLmHead(HomBertEncoder *e) {
  if (e->lmHead)
    return 0;
  {
    const int64_t M = int64_t(e->batch) * e->seq;
    if (!chooseGemm(e, M, e->hidden, e->hidden, e->geluForm == 1 ? 2 : 1, 0.0f,
                    e->roleLayout[4], &e->cTransform) ||
        !chooseGemm(e, M, e->vocab, e->hidden, 0, 0.0f, e->roleLayout[5],
                    &e->cDecoder))
      return -1;
  }
  e->wTransform.m = alloc3DMemRefNVGPUF16(1, e->hidden, e->hidden);
  e->wDecoder.m = e->cDecoder.nk
                      ? alloc3DMemRefNVGPUF16(1, e->vocab, e->hidden)
                      : alloc3DMemRefNVGPUF16(1, e->hidden, e->vocab);
  e->t.m = alloc3DMemRefNVGPUF16(e->batch, e->seq, e->hidden);
  e->logits.m = alloc3DMemRefNVGPUF16(e->batch, e->seq, e->vocab);
  if (!e->wTransform.data() || !e->wDecoder.data() || !e->t.data() ||
      !e->logits.data())
    return -1;
  e->lmHead = true;
  return 0;
}

// Switches the call list to the variant with folded layer norms (see
// callList).  Call after every weight has been uploaded (the column sums of
// Wqkv and W1 are computed here) and before capturing a graph.  Needs all four
// GEMM roles on row-major weights and the erf form of GELU; the LM head keeps
// its own layer norm.  Returns 0, or -1 when the configuration does not allow
// it (nothing changes then).
DRV_EXPORT int homBertFoldLayernorm(HomBertEncoder *e) {
  if (e->foldLn)
    return 0;
  if (e->cQkv.nk || e->cOut.nk || e->cFfn1.nk || e->cFfn2.nk ||
      e->geluForm != 0 || e->gemmMode == 0 || e->hidden % 8 != 0 ||
      e->ffn % 8 != 0) {
    fprintf(stderr, "hom_bert_driver: folded layer norms need row-major "
                    "weights for every GEMM role and the erf form of GELU\n");
    return -1;
  }
  const int64_t M = int64_t(e->batch) * e->seq;
  const int32_t pOut = homFoldedLayernormPieces(M, e->hidden, e->hidden, 0, 0);
  const int32_t pFfn2 = homFoldedLayernormPieces(M, e->hidden, e->ffn, 0, 0);
  if (pOut != pFfn2 || pOut < 1)
    return -1; // (both depend on M and N only)
  bool ok = true;
  for (float *&q : e->rowSums)
    ok = ok && hipOk(hipMalloc(reinterpret_cast<void **>(&q),
                               size_t(pOut) * size_t(M) * 2 * sizeof(float)),
                     "hipMalloc");
  void *prev = homGetStream();
  homSetStream(e->stream);
  for (int l = 0; l < e->layers && ok; l++) {
    float *q = nullptr, *f = nullptr;
    ok = hipOk(hipMalloc(reinterpret_cast<void **>(&q), size_t(3) * e->hidden * 4),
               "hipMalloc") &&
         hipOk(hipMalloc(reinterpret_cast<void **>(&f), size_t(e->ffn) * 4),
               "hipMalloc");
    e->colSumQkv.push_back(q);
    e->colSumW1.push_back(f);
    if (ok) {
      const LayerWeights &w = e->w[size_t(l)];
      homColumnSumsF16(w.wqkv.m.rank, w.wqkv.m.descriptor, q);
      homColumnSumsF16(w.w1.m.rank, w.w1.m.descriptor, f);
    }
  }
  homSetStream(prev);
  ok = ok && hipOk(hipStreamSynchronize(e->stream), "hipStreamSynchronize");
  if (!ok)
    return -1;
  e->foldPieces = pOut;
  e->foldLn = true;
  return 0;
}

DRV_EXPORT void homBertDestroy(HomBertEncoder *e) {
  if (!e)
    return;
  if (e->graphExec)
    (void)hipGraphExecDestroy(e->graphExec);
  if (e->graph)
    (void)hipGraphDestroy(e->graph);
  if (e->stream) {
    (void)hipStreamSynchronize(e->stream);
    homReleaseStreamScratch(e->stream);
    (void)hipStreamDestroy(e->stream);
  }
  if (e->evStart)
    (void)hipEventDestroy(e->evStart);
  if (e->evStop)
    (void)hipEventDestroy(e->evStop);
  for (auto &w : e->w) {
    w.wqkv.release();
    w.wo.release();
    w.w1.release();
    w.w2.release();
  }
  for (float *q : e->colSumQkv)
    (void)hipFree(q);
  for (float *q : e->colSumW1)
    (void)hipFree(q);
  for (float *q : e->rowSums)
    if (q)
      (void)hipFree(q);
  for (Tensor *t : {&e->wordEmb, &e->posType, &e->ids, &e->mask, &e->cu, &e->h,
                    &e->emb, &e->qkv, &e->attn, &e->f, &e->wTransform,
                    &e->wDecoder, &e->t, &e->logits})
    t->release();
  delete e;
}

// which: 0 Wqkv, 1 Wo, 2 W1, 3 W2 (layer >= 0); 4 word embeddings, 5 position +
// token-type rows, 6 LM-head transform weight, 7 LM-head decoder weight (layer
// ignored; 6 and 7 after homBertEnableLmHead).  `host` holds fp16 values in the layout the
// tensor was allocated with ([K, N] row-major, or [N, K] when gemmMode == 0).
DRV_EXPORT int homBertUpload(HomBertEncoder *e, int layer, int which,
                             const void *host, int64_t numel) {
  Tensor *t = nullptr;
  if (which <= 3) {
    if (layer < 0 || layer >= e->layers)
      return -1;
    LayerWeights &w = e->w[size_t(layer)];
    t = which == 0 ? &w.wqkv : which == 1 ? &w.wo : which == 2 ? &w.w1 : &w.w2;
  } else if (which <= 5) {
    t = which == 4 ? &e->wordEmb : &e->posType;
  } else {
    if (!e->lmHead || which > 7)
      return -1;
    t = which == 6 ? &e->wTransform : &e->wDecoder;
  }
  int64_t expect = 1;
  for (int64_t i = 0; i < t->m.rank; i++)
    expect *= hom_memref_sizes(t->m.descriptor)[i];
  if (expect != numel) {
    fprintf(stderr, "hom_bert_driver: upload of %lld values into a tensor of "
                    "%lld\n", (long long)numel, (long long)expect);
    return -2;
  }
  return hipOk(hipMemcpy(t->data(), host, size_t(numel) * 2,
                         hipMemcpyHostToDevice),
               "hipMemcpy")
             ? 0
             : -3;
}

// Inputs: token ids and 0/1 mask (int64 [b, s]); `hidden` (fp16 [b, s, H]) may
// be given instead of ids to start from precomputed embeddings.
DRV_EXPORT int homBertSetInputs(HomBertEncoder *e, const int64_t *ids,
                                const int64_t *mask, const void *hidden) {
  const size_t n = size_t(e->batch) * e->seq;
  if (ids && !hipOk(hipMemcpy(e->ids.data(), ids, n * 8, hipMemcpyHostToDevice),
                    "hipMemcpy ids"))
    return -1;
  if (mask &&
      !hipOk(hipMemcpy(e->mask.data(), mask, n * 8, hipMemcpyHostToDevice),
             "hipMemcpy mask"))
    return -1;
  if (hidden && !hipOk(hipMemcpy(e->h.data(), hidden, n * e->hidden * 2,
                                 hipMemcpyHostToDevice),
                       "hipMemcpy hidden"))
    return -1;
  return 0;
}

// One eager forward on the driver's stream; returns after enqueueing.
DRV_EXPORT void homBertForward(HomBertEncoder *e, int fromIds) {
  void *prev = homGetStream();
  homSetStream(e->stream);
  callList(e, fromIds);
  homSetStream(prev);
}

// Capture the call list once (after one eager run has sized the library's
// scratch buffers) and keep the instantiated graph.
DRV_EXPORT int homBertCapture(HomBertEncoder *e, int fromIds) {
  homBertForward(e, fromIds);
  if (!hipOk(hipStreamSynchronize(e->stream), "hipStreamSynchronize"))
    return -1;
  if (e->graphExec) {
    (void)hipGraphExecDestroy(e->graphExec);
    e->graphExec = nullptr;
  }
  if (e->graph) {
    (void)hipGraphDestroy(e->graph);
    e->graph = nullptr;
  }
  void *prev = homGetStream();
  homSetStream(e->stream);
  bool ok = hipOk(hipStreamBeginCapture(e->stream, hipStreamCaptureModeRelaxed),
                  "hipStreamBeginCapture");
  if (ok) {
    callList(e, fromIds);
    ok = hipOk(hipStreamEndCapture(e->stream, &e->graph), "hipStreamEndCapture");
  }
  homSetStream(prev);
  if (!ok)
    return -1;
  if (!hipOk(hipGraphInstantiate(&e->graphExec, e->graph, nullptr, nullptr, 0),
             "hipGraphInstantiate"))
    return -1;
  return 0;
}

DRV_EXPORT int homBertReplay(HomBertEncoder *e) {
  if (!e->graphExec)
    return -1;
  return hipOk(hipGraphLaunch(e->graphExec, e->stream), "hipGraphLaunch") ? 0
                                                                          : -1;
}

// The stream the encoder's calls are enqueued on (a hipStream_t).
DRV_EXPORT void *homBertGetStream(HomBertEncoder *e) {
  return static_cast<void *>(e->stream);
}

DRV_EXPORT int homBertSync(HomBertEncoder *e) {
  return hipOk(hipStreamSynchronize(e->stream), "hipStreamSynchronize") ? 0 : -1;
}

// Copy the encoder output (the hidden-state buffer, updated in place) to host.
DRV_EXPORT int homBertGetOutput(HomBertEncoder *e, void *host) {
  if (homBertSync(e) != 0)
    return -1;
  const size_t n = size_t(e->batch) * e->seq * e->hidden;
  return hipOk(hipMemcpy(host, e->h.data(), n * 2, hipMemcpyDeviceToHost),
               "hipMemcpy out")
             ? 0
             : -1;
}

// Copy the masked-LM logits [b, s, vocab] to host.
DRV_EXPORT int homBertGetLogits(HomBertEncoder *e, void *host) {
  if (!e->lmHead || homBertSync(e) != 0)
    return -1;
  const size_t n = size_t(e->batch) * e->seq * e->vocab;
  return hipOk(hipMemcpy(host, e->logits.data(), n * 2, hipMemcpyDeviceToHost),
               "hipMemcpy logits")
             ? 0
             : -1;
}

// Time `steps` forwards after `warmup` untimed ones, bracketed by events on the
// driver's stream (the reference's protocol: bert.cu:95-127).  useGraph != 0
// replays the captured graph.  Returns mean milliseconds per forward, < 0 on
// error.  Inputs stay resident; every forward recomputes from the token ids.
DRV_EXPORT double homBertTime(HomBertEncoder *e, int steps, int warmup,
                              int useGraph, int fromIds) {
  if (useGraph && !e->graphExec && homBertCapture(e, fromIds) != 0)
    return -1.0;
  for (int i = 0; i < warmup; i++) {
    if (useGraph)
      homBertReplay(e);
    else
      homBertForward(e, fromIds);
  }
  if (homBertSync(e) != 0)
    return -1.0;
  (void)hipEventRecord(e->evStart, e->stream);
  for (int i = 0; i < steps; i++) {
    if (useGraph)
      homBertReplay(e);
    else
      homBertForward(e, fromIds);
  }
  (void)hipEventRecord(e->evStop, e->stream);
  if (!hipOk(hipEventSynchronize(e->evStop), "hipEventSynchronize"))
    return -1.0;
  float ms = 0.f;
  (void)hipEventElapsedTime(&ms, e->evStart, e->evStop);
  return double(ms) / double(steps > 0 ? steps : 1);
}

DRV_EXPORT void homBertGetGemmChoices(HomBertEncoder *e, int32_t *out8) {
  const GemmChoice *c[4] = {&e->cQkv, &e->cOut, &e->cFfn1, &e->cFfn2};
  for (int i = 0; i < 4; i++) {
    out8[2 * i] = c[i]->gemmNum;
    out8[2 * i + 1] = c[i]->splitK;
  }
}

// Pins the manifest kernel (1-based, as cutlassGemmF16 takes it) and split-K
// factor of one GEMM role: 0 QKV, 1 output projection, 2 FFN1, 3 FFN2.  What a
// compiled module carries as constants; here it lets the autotuner time
// candidates inside the encoder graph, where operands arrive cold from the
// previous kernel.  A captured graph must be captured again afterwards.
DRV_EXPORT int homBertSetGemmChoice(HomBertEncoder *e, int role,
                                    int32_t gemmNum, int32_t splitK) {
  GemmChoice *c[4] = {&e->cQkv, &e->cOut, &e->cFfn1, &e->cFfn2};
  if (role < 0 || role > 3 || gemmNum < 1 || gemmNum > homGemmManifestSize() ||
      splitK < 1)
    return -1;
  if (c[role]->nk)
    return -2; // the role's weight is [N, K]: it runs through nvteGemmF16
  c[role]->gemmNum = gemmNum;
  c[role]->splitK = splitK;
  return 0;
}

// ---- single-operator timing through the boundary -------------------------
// Each helper enqueues `iters` back-to-back calls of one entry point between
// two events on a private stream, behind a warm-up (Timer::warm), and returns
// mean milliseconds per call.

namespace {
struct Timer {
  hipStream_t s = nullptr;
  hipEvent_t a = nullptr, b = nullptr;
  void *prev = nullptr;
  bool ok = false;
  Timer() {
    ok = hipOk(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "stream") &&
         hipOk(hipEventCreate(&a), "event") && hipOk(hipEventCreate(&b), "event");
    prev = homGetStream();
    homSetStream(s);
  }
  ~Timer() {
    homSetStream(prev);
    if (a)
      (void)hipEventDestroy(a);
    if (b)
      (void)hipEventDestroy(b);
    if (s) {
      (void)hipStreamSynchronize(s);
      homReleaseStreamScratch(s);
      (void)hipStreamDestroy(s);
    }
  }
  // Untimed calls before the timed ones: at least `warmup`, and as many as it
  // takes to keep the GPU busy for kMinWarmMs.  After an idle period (the
  // uploads that precede a timing loop are one) the first tens of
  // milliseconds of launches run slower than the steady state: 10.1 us per
  // launch against 8.7 us for the 1024 x 3072 x 768 GEMM.
  static constexpr double kMinWarmMs = 150.0;
  template <typename F> bool warm(F &&fn, int warmup) {
    const auto t0 = std::chrono::steady_clock::now();
    const int batch = warmup > 10 ? warmup : 10;
    for (;;) {
      for (int i = 0; i < batch; i++)
        fn();
      if (!hipOk(hipStreamSynchronize(s), "sync"))
        return false;
      const double ms = std::chrono::duration<double, std::milli>(
                            std::chrono::steady_clock::now() - t0)
                            .count();
      if (ms >= kMinWarmMs)
        return true;
    }
  }
  template <typename F> double run(F &&fn, int iters, int warmup) {
    if (!ok || !warm(fn, warmup))
      return -1.0;
    (void)hipEventRecord(a, s);
    for (int i = 0; i < iters; i++)
      fn();
    (void)hipEventRecord(b, s);
    if (!hipOk(hipEventSynchronize(b), "event sync"))
      return -1.0;
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, a, b);
    return double(ms) / double(iters > 0 ? iters : 1);
  }
  // The same calls as kernel nodes of a HIP graph: `perGraph` calls are
  // captured once and the graph is replayed `replays` times between the
  // events.  Inside a graph a dependent launch costs less than on a stream,
  // and a graph is how the encoder's call list runs.
  template <typename F>
  double runGraph(F &&fn, int perGraph, int replays, int warmup) {
    if (!ok)
      return -1.0;
    fn(); // sizes whatever scratch the call needs before the capture
    if (!hipOk(hipStreamSynchronize(s), "sync"))
      return -1.0;
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    if (!hipOk(hipStreamBeginCapture(s, hipStreamCaptureModeRelaxed), "capture"))
      return -1.0;
    for (int i = 0; i < perGraph; i++)
      fn();
    double out = -1.0;
    if (hipOk(hipStreamEndCapture(s, &g), "end capture") &&
        hipOk(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0), "instantiate")) {
      if (warm([&] { (void)hipGraphLaunch(ge, s); }, warmup)) {
        (void)hipEventRecord(a, s);
        for (int i = 0; i < replays; i++)
          (void)hipGraphLaunch(ge, s);
        (void)hipEventRecord(b, s);
        if (hipOk(hipEventSynchronize(b), "event sync")) {
          float ms = 0.f;
          (void)hipEventElapsedTime(&ms, a, b);
          out = double(ms) / double(replays > 0 ? replays : 1) /
                double(perGraph > 0 ? perGraph : 1);
        }
      }
    }
    if (ge)
      (void)hipGraphExecDestroy(ge);
    if (g)
      (void)hipGraphDestroy(g);
    return out;
  }
};

void fillRandomF16(void *dev, int64_t numel, float scale, uint32_t seed) {
  std::vector<uint16_t> host(static_cast<size_t>(numel));
  uint32_t x = seed * 2654435761u + 12345u;
  for (auto &v : host) {
    // xorshift; sum of 4 uniforms, roughly normal, scaled
    float acc = 0.f;
    for (int i = 0; i < 4; i++) {
      x ^= x << 13;
      x ^= x >> 17;
      x ^= x << 5;
      acc += float(x & 0xffff) / 65536.0f - 0.5f;
    }
    _Float16 h = _Float16(acc * 1.7320508f * scale);
    memcpy(&v, &h, 2);
  }
  (void)hipMemcpy(dev, host.data(), size_t(numel) * 2, hipMemcpyHostToDevice);
}
} // namespace

// What the matrix cores deliver when nothing else is in the way: every
// wavefront (two per SIMD, the occupancy of the large GEMM tiles) issues
// v_mfma_f32_32x32x16_f16 back to back on operands that never leave its
// registers, four independent accumulator blocks, no memory access inside the
// loop.  VALU_PER_MFMA independent fp32 FMAs are placed behind every MFMA.
typedef _Float16 ProbeHalf8 __attribute__((ext_vector_type(8)));
typedef float ProbeFloat16 __attribute__((ext_vector_type(16)));
template <int VALU_PER_MFMA>
__global__ __launch_bounds__(512) void mfmaCeilingKernel(const _Float16 *in,
                                                         float *out, int iters) {
  ProbeHalf8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = in[(threadIdx.x * 8 + i) & 4095];
    b[i] = in[4096 + ((threadIdx.x * 8 + i) & 4095)];
  }
  ProbeFloat16 acc[4] = {};
  float x[8];
  for (int i = 0; i < 8; ++i)
    x[i] = float(in[(i + threadIdx.x) & 4095]);
  const float c = float(in[3]) * 1e-3f + 1.0f, d = float(in[5]);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      acc[j & 3] =
          __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j & 3], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
      for (int v = 0; v < VALU_PER_MFMA; ++v) {
        const int k = (j * VALU_PER_MFMA + v) & 7;
        x[k] = fmaf(x[k], c, d);
      }
      if (VALU_PER_MFMA)
        __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);
    }
  }
  float s = 0;
  for (int i = 0; i < 8; ++i)
    s += x[i];
  for (int k = 0; k < 4; ++k)
    for (int i = 0; i < 16; ++i)
      s += acc[k][i];
  out[blockIdx.x * 512 + threadIdx.x] = s;
}

// TFLOP/s of that loop on one workgroup of 8 wavefronts per CU.
// randomOperands: 0 = all operands zero, 1 = values in [-1, 1).  valuPerMfma:
// 0, 4 or 8.  Negative on error.
DRV_EXPORT double homMfmaCeilingProbe(int randomOperands, int valuPerMfma) {
  const int n = 8192;
  Tensor in, out;
  in.m = alloc3DMemRefNVGPUF16(1, 1, n);
  out.m = alloc3DMemRefNVGPUF16(1, 512, 2 * 512); // 256 * 512 floats
  if (!in.data() || !out.data())
    return -1.0;
  if (randomOperands)
    fillRandomF16(in.data(), n, 0.5f, 11);
  else
    (void)hipMemset(in.data(), 0, size_t(n) * 2);
  const int iters = 4000, launches = 5;
  double tflops = -1.0;
  {
    Timer t;
    auto call = [&] {
      const _Float16 *src = static_cast<const _Float16 *>(in.data());
      float *dst = static_cast<float *>(out.data());
      if (valuPerMfma >= 8)
        mfmaCeilingKernel<8><<<256, 512, 0, t.s>>>(src, dst, iters);
      else if (valuPerMfma >= 4)
        mfmaCeilingKernel<4><<<256, 512, 0, t.s>>>(src, dst, iters);
      else
        mfmaCeilingKernel<0><<<256, 512, 0, t.s>>>(src, dst, iters);
    };
    const double ms = t.run(call, launches, 2);
    // 256 workgroups x 8 wavefronts x 16 MFMAs of 32 x 32 x 16 per iteration
    if (ms > 0)
      tflops = 256.0 * 8 * 16 * iters * (2.0 * 32 * 32 * 16) / (ms * 1e-3) / 1e12;
  }
  in.release();
  out.release();
  return tflops;
}

// What one kernel node of a replayed graph costs when the kernel does nothing:
// `nodes` empty kernels of `groups` workgroups captured into one graph, ms per
// node over `replays` replays.  The floor under every kernel of the encoder's
// 88-launch chain.  Negative on error.
namespace {
__global__ void emptyNodeKernel() {}
} // namespace
DRV_EXPORT double homTimeEmptyGraphNodes(int nodes, int groups, int replays) {
  if (nodes < 1 || groups < 1 || replays < 1)
    return -1.0;
  Timer t;
  return t.runGraph([&] { emptyNodeKernel<<<groups, 256, 0, t.s>>>(); }, nodes,
                    replays, 5);
}

// D = act(A.B + bias) with bias broadcast as a [1,1,N] C (useBias) or beta = 0.
// gemmNum is 1-based (0 = library picks); returns ms per call.  inGraph != 0:
// 100 calls per captured graph, iters / 100 replays.
static double timeGemm(int64_t M, int64_t N, int64_t K, int64_t act,
                       int useBias, int32_t gemmNum, int32_t splitK, int iters,
                       int warmup, int inGraph, bool zeroOperands = false) {
  Tensor a, b, c, d;
  a.m = alloc3DMemRefNVGPUF16(1, int32_t(M), int32_t(K));
  b.m = alloc3DMemRefNVGPUF16(1, int32_t(K), int32_t(N));
  c.m = alloc3DMemRefNVGPUF16(1, 1, int32_t(N));
  d.m = alloc3DMemRefNVGPUF16(1, int32_t(M), int32_t(N));
  if (zeroOperands) {
    (void)hipMemset(a.data(), 0, size_t(M * K) * 2);
    (void)hipMemset(b.data(), 0, size_t(K * N) * 2);
    (void)hipMemset(c.data(), 0, size_t(N) * 2);
  } else {
    fillRandomF16(a.data(), M * K, 1.0f, 1);
    fillRandomF16(b.data(), K * N, 0.02f, 2);
    fillRandomF16(c.data(), N, 0.02f, 3);
  }
  double ms;
  {
    Timer t;
    auto call = [&] {
      cutlassGemmF16(3, a.m.descriptor, false, 3, b.m.descriptor, false, 3,
                     useBias ? c.m.descriptor : d.m.descriptor, 3,
                     d.m.descriptor, act, 1.0f, useBias ? 1.0f : 0.0f, gemmNum,
                     splitK);
    };
    ms = inGraph ? t.runGraph(call, 100, (iters + 99) / 100, (warmup + 99) / 100)
                 : t.run(call, iters, warmup);
  }
  a.release();
  b.release();
  c.release();
  d.release();
  return ms;
}

DRV_EXPORT double homTimeGemm(int64_t M, int64_t N, int64_t K, int64_t act,
                              int useBias, int32_t gemmNum, int32_t splitK,
                              int iters, int warmup) {
  return timeGemm(M, N, K, act, useBias, gemmNum, splitK, iters, warmup, 0);
}

// The same kernel on operands that are all zero: identical instructions and
// memory traffic, no switching in the data paths.  What it gains over
// homTimeGemm is what the chip's power management takes from the kernel on
// real data.
DRV_EXPORT double homTimeGemmZeroOperands(int64_t M, int64_t N, int64_t K,
                                          int64_t act, int useBias,
                                          int32_t gemmNum, int32_t splitK,
                                          int iters, int warmup) {
  return timeGemm(M, N, K, act, useBias, gemmNum, splitK, iters, warmup, 0,
                  true);
}

DRV_EXPORT double homTimeGemmInGraph(int64_t M, int64_t N, int64_t K,
                                     int64_t act, int useBias, int32_t gemmNum,
                                     int32_t splitK, int iters, int warmup) {
  return timeGemm(M, N, K, act, useBias, gemmNum, splitK, iters, warmup, 1);
}

// Same through nvteGemmF16 (B given as [1, N, K]); the library picks the kernel.
DRV_EXPORT double homTimeGemmNvte(int64_t M, int64_t N, int64_t K, int64_t act,
                                  int iters, int warmup) {
  Tensor a, b, d;
  a.m = alloc3DMemRefNVGPUF16(1, int32_t(M), int32_t(K));
  b.m = alloc3DMemRefNVGPUF16(1, int32_t(N), int32_t(K));
  d.m = alloc3DMemRefNVGPUF16(1, int32_t(M), int32_t(N));
  fillRandomF16(a.data(), M * K, 1.0f, 1);
  fillRandomF16(b.data(), K * N, 0.02f, 2);
  double ms;
  {
    Timer t;
    ms = t.run(
        [&] {
          nvteGemmF16(3, a.m.descriptor, false, 3, b.m.descriptor, true, 3,
                      d.m.descriptor, 3, d.m.descriptor, act, 1.0f, 0.0f, 0, 0);
        },
        iters, warmup);
  }
  a.release();
  b.release();
  d.release();
  return ms;
}

// In-place layer norm (reference form) when fused == 0; residual add + affine
// layer norm (homAddLayernormF16) when fused != 0.  The calls walk round-robin
// over `sets` independent sets of tensors (x; x, residual and output when
// fused).  With one set the tensors stay in the 256 MB last-level cache from
// launch to launch whenever they fit, and the figure is a cache rate; with
// sets whose total size is several times that cache every launch reads from
// and writes to HBM.
DRV_EXPORT double homTimeLayernormRotating(int64_t rows, int64_t hidden,
                                           int fused, int sets, int iters,
                                           int warmup) {
  if (sets < 1)
    sets = 1;
  const size_t nSets = size_t(sets), nFused = fused ? nSets : 0;
  std::vector<Tensor> x(nSets), r(nFused), o(nFused);
  Tensor g, bt;
  g.m = alloc3DMemRefNVGPUF16(1, 1, int32_t(hidden));
  bt.m = alloc3DMemRefNVGPUF16(1, 1, int32_t(hidden));
  fillRandomF16(g.data(), hidden, 0.02f, 6);
  fillRandomF16(bt.data(), hidden, 0.02f, 7);
  const size_t bytes = size_t(rows) * size_t(hidden) * 2;
  bool ok = g.data() && bt.data();
  for (int i = 0; i < sets && ok; i++) {
    x[size_t(i)].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
    ok = x[size_t(i)].data() != nullptr;
    if (fused && ok) {
      r[size_t(i)].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
      o[size_t(i)].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
      ok = r[size_t(i)].data() && o[size_t(i)].data();
    }
    if (!ok)
      break;
    if (i == 0) {
      fillRandomF16(x[0].data(), rows * hidden, 1.0f, 4);
      if (fused)
        fillRandomF16(r[0].data(), rows * hidden, 1.0f, 5);
    } else {
      (void)hipMemcpy(x[size_t(i)].data(), x[0].data(), bytes,
                      hipMemcpyDeviceToDevice);
      if (fused)
        (void)hipMemcpy(r[size_t(i)].data(), r[0].data(), bytes,
                        hipMemcpyDeviceToDevice);
    }
  }
  double ms = -1.0;
  if (ok) {
    Timer t;
    int next = 0;
    ms = t.run(
        [&] {
          const size_t i = size_t(next);
          next = next + 1 == sets ? 0 : next + 1;
          if (fused)
            homAddLayernormF16(3, x[i].m.descriptor, 3, r[i].m.descriptor, 3,
                               g.m.descriptor, 3, bt.m.descriptor, 3,
                               o[i].m.descriptor, 1e-12f);
          else
            nvteLayernormF16(3, x[i].m.descriptor, 1e-12f);
        },
        iters, warmup);
  }
  for (auto *v : {&x, &r, &o})
    for (Tensor &t : *v)
      t.release();
  g.release();
  bt.release();
  return ms;
}

DRV_EXPORT double homTimeLayernorm(int64_t rows, int64_t hidden, int fused,
                                   int iters, int warmup) {
  return homTimeLayernormRotating(rows, hidden, fused, 1, iters, warmup);
}

// Packed-QKV attention with per-sequence valid lengths `lens` (host, int32[bs]).
DRV_EXPORT double homTimeAttention(int64_t bs, int64_t seq, int64_t heads,
                                   const int32_t *lens, int iters, int warmup) {
  const int64_t hd = heads * 64;
  Tensor qkv, out, cu;
  qkv.m = alloc3DMemRefNVGPUF16(int32_t(bs), int32_t(seq), int32_t(3 * hd));
  out.m = alloc3DMemRefNVGPUF16(int32_t(bs), int32_t(seq), int32_t(hd));
  cu.m = alloc1DMemRefNVGPUI32(int32_t(bs + 1));
  fillRandomF16(qkv.data(), bs * seq * 3 * hd, 1.0f, 8);
  std::vector<int32_t> cuHost(size_t(bs + 1), 0);
  for (int64_t i = 0; i < bs; i++)
    cuHost[size_t(i + 1)] = cuHost[size_t(i)] + lens[i];
  (void)hipMemcpy(cu.data(), cuHost.data(), size_t(bs + 1) * 4,
                  hipMemcpyHostToDevice);
  double ms;
  {
    Timer t;
    ms = t.run(
        [&] {
          nvteBertAttentionF16(3, qkv.m.descriptor, 1, cu.m.descriptor, 3,
                               out.m.descriptor, 0.125f, heads);
        },
        iters, warmup);
  }
  qkv.release();
  out.release();
  cu.release();
  return ms;
}

// out = a + b over `sets` independent (a, b, out) triples walked round-robin
// (see homTimeLayernormRotating for what the number of sets decides).
DRV_EXPORT double homTimeElementwiseAddRotating(int64_t rows, int64_t hidden,
                                                int sets, int iters,
                                                int warmup) {
  if (sets < 1)
    sets = 1;
  const size_t nSets = size_t(sets);
  std::vector<Tensor> a(nSets), b(nSets), o(nSets);
  const size_t bytes = size_t(rows) * size_t(hidden) * 2;
  bool ok = true;
  for (int i = 0; i < sets && ok; i++) {
    const size_t k = size_t(i);
    a[k].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
    b[k].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
    o[k].m = alloc3DMemRefNVGPUF16(1, int32_t(rows), int32_t(hidden));
    ok = a[k].data() && b[k].data() && o[k].data();
    if (!ok)
      break;
    if (i == 0) {
      fillRandomF16(a[0].data(), rows * hidden, 1.0f, 9);
      fillRandomF16(b[0].data(), rows * hidden, 1.0f, 10);
    } else {
      (void)hipMemcpy(a[k].data(), a[0].data(), bytes, hipMemcpyDeviceToDevice);
      (void)hipMemcpy(b[k].data(), b[0].data(), bytes, hipMemcpyDeviceToDevice);
    }
  }
  double ms = -1.0;
  if (ok) {
    Timer t;
    int next = 0;
    ms = t.run(
        [&] {
          const size_t i = size_t(next);
          next = next + 1 == sets ? 0 : next + 1;
          thrustElementwiseAddF16(3, a[i].m.descriptor, 3, b[i].m.descriptor, 3,
                                  o[i].m.descriptor);
        },
        iters, warmup);
  }
  for (auto *v : {&a, &b, &o})
    for (Tensor &t : *v)
      t.release();
  return ms;
}

DRV_EXPORT double homTimeElementwiseAdd(int64_t rows, int64_t hidden, int iters,
                                        int warmup) {
  return homTimeElementwiseAddRotating(rows, hidden, 1, iters, warmup);
}
