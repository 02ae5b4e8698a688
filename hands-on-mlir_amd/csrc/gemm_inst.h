// Explicit instantiation helpers for the gemm_inst_*.hip translation units:
// each defines HOM_INST_FAMILY to the family it owns before including this
// file and gemm_manifest.inc, and gets the six launch functions (three
// epilogues x two B layouts) of every tile of that family.
#pragma once

#define HOM_INST_EPILOGUES(FN, ...)                                            \
  template Status FN<__VA_ARGS__, 0, false>(const GemmProblem &, hipStream_t); \
  template Status FN<__VA_ARGS__, 0, true>(const GemmProblem &, hipStream_t);  \
  template Status FN<__VA_ARGS__, 1, false>(const GemmProblem &, hipStream_t); \
  template Status FN<__VA_ARGS__, 1, true>(const GemmProblem &, hipStream_t);  \
  template Status FN<__VA_ARGS__, 2, false>(const GemmProblem &, hipStream_t); \
  template Status FN<__VA_ARGS__, 2, true>(const GemmProblem &, hipStream_t);

// the same for the register-staged family's DMA variant (launchPipe<..., true>)
#define HOM_INST_EPILOGUES_DMA(FN, ...)                                        \
  template Status FN<__VA_ARGS__, 0, false, true>(const GemmProblem &,         \
                                                  hipStream_t);                \
  template Status FN<__VA_ARGS__, 0, true, true>(const GemmProblem &,          \
                                                 hipStream_t);                 \
  template Status FN<__VA_ARGS__, 1, false, true>(const GemmProblem &,         \
                                                  hipStream_t);                \
  template Status FN<__VA_ARGS__, 1, true, true>(const GemmProblem &,          \
                                                 hipStream_t);                 \
  template Status FN<__VA_ARGS__, 2, false, true>(const GemmProblem &,         \
                                                  hipStream_t);                \
  template Status FN<__VA_ARGS__, 2, true, true>(const GemmProblem &,          \
                                                 hipStream_t);

#define HOM_DMA_TILE(...)
#define HOM_PIPE_TILE_Q(...)
#define HOM_PIPE_TILE_A(...)
#define HOM_PIPE_TILE_B(...)
#define HOM_PIPE_TILE_C(...)
#define HOM_PIPE_TILE_D(...)
#define HOM_FINE_TILE(...)
#define HOM_STAGED_TILE(...)
