// Device-side building blocks shared by the fp16 GEMM kernel families
// (gemm_dma.h, gemm_pipe.h, gemm_staged.h) and their launch plumbing.
//
//   D = epilogue(alpha * A.B + beta * C)
//   A [M, K] row-major; B [K, N] row-major (or [N, K] when pre-transposed);
//   C, D [M, N] row-major, D may alias C.
//
// These kernels replace the CUTLASS GemmUniversal instances the reference
// generates (python/gemm_generator.py:237-278, python/hom_manifest.py:503-533)
// and the cuBLASLt call behind nvteGemmF16
// (include/NVGPUKernels/GemmRunner.h:404-425).
//
// Common structure
//  * one workgroup of WM x WN wavefronts computes a BM x BN tile of D; every
//    wavefront owns a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks
//    (v_mfma_f32_32x32x16_f16: 64 lanes x 8 halves per operand, 16 fp32
//    accumulators per lane);
//  * the MFMA is issued with the operands swapped (B fragment first), i.e. it
//    produces the transposed block, so each lane ends up with 4 consecutive
//    columns of one row of D and the epilogue can use 64-bit accesses;
//  * split-K: gridDim.y slices of K each store their fp32 partial tile to a
//    workspace; a second, small kernel sums the slices in slice order
//    (deterministic, fp32) and runs the epilogue.  Nothing spins or fences.
//    Optionally (pipe kernels, slices of a tile on one XCD) the slice that
//    finishes last forms the same sum inside the kernel: arriveAtTile();
//  * workgroup ids are remapped so that each of the 8 XCDs (which receive
//    consecutive ids round-robin and have private L2s) works on a contiguous
//    run of tiles.
//
// The kernel templates live in headers and are instantiated explicitly in the
// gemm_inst_*.hip translation units (one per family / size class, so that they
// compile in parallel); gemm.hip holds the manifest table that refers to the
// launch functions.
#pragma once

#include "cross_lane.h"
#include "kernels.h"
#include "store_policy.h"

#include <algorithm>
#include <type_traits>
#include <utility>

namespace hom {
namespace gemmk {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), unrolled.
template <class F, int... I>
__device__ __forceinline__ void staticForImpl(F &&f,
                                              std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F> __device__ __forceinline__ void staticFor(F &&f) {
  staticForImpl(f, std::make_integer_sequence<int, N>{});
}

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kNumXcd = 8;

#define HOM_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

struct GemmParams {
  const _Float16 *A;
  const _Float16 *B;
  const _Float16 *C;
  _Float16 *D;
  float *workspace; // split-K partial tiles (null when gridDim.y == 1)
  // In-kernel split-K reduction (null: a second kernel sums the slices): one
  // arrival word per tile, and the host-visible word that reports slices of
  // one tile found on different XCDs.
  unsigned long long *tileArrivals;
  unsigned int *misplaced;
  int M, N, K;
  int64_t lda, ldb, ldc, ldd;
  int cRowPeriod;
  float alpha, beta;
  int tilesM, tilesN;
  int kTilesPerSlice;
  // Tile order, prepared on the host so that a workgroup finds its tile with a
  // few scalar instructions (tileCoordsFast): tiles per XCD (quotient and
  // remainder), floor(2^32 / d) for the divisor of the tile walk, the number of
  // full groups of kGroupM tile rows and the rows of the last group.
  int xcdQ, xcdR;
  uint32_t groupMagic;
  uint32_t cRowMagic; // floor(2^32 / cRowPeriod)
  int fullGroups, lastRows;
  // epilogueFastMode() evaluated on the host for the whole launch
  int epiMode;
  // layer-norm pair (kEpiRowStats / kEpiRowAffine kernels only)
  float *rowStatPartials;
  const _Float16 *rowScale;
  const _Float16 *rowShift;
  const float *colSum;
  int colSumSlices;
  // folded layer norm (kEpiFold* kernels only): partial (sum, sum of squares)
  // pairs [foldPieces][M] of the rows a layer norm is folded away from -- the
  // rows of A (kEpiFoldA, kEpiFoldAGelu) or of C (kEpiFoldCStats) -- the
  // reciprocal of their length and the layer norm's epsilon.  Null: the rows
  // are used as they are.
  const float *foldStats;
  int foldPieces;
  float foldInvN, foldEps;
};

// Epilogue codes beyond the three activations of the manifest kernels: linear
// output plus row-statistic partial sums, and linear output of a per-row
// affine transform of A folded into the accumulator.
constexpr int kEpiRowStats = 3;
constexpr int kEpiRowAffine = 4;
// A layer norm (no affine parameters) folded into the GEMMs on either side of
// it, with its statistics travelling as the fp32 partial sums that the
// producing GEMM's epilogue wrote (nothing in between):
//   kEpiFoldA       D = alpha (LN(A) . B) + beta C
//   kEpiFoldAGelu   D = GELU_erf(alpha (LN(A) . B) + beta C)
//   kEpiFoldCStats  D = alpha (A . B) + beta LN(C), plus the partial sums of
//                   the stored D (for the next folded layer norm)
// LN(A) . B is evaluated as rstd_m (A . B) - mu_m rstd_m colsum(B), see
// kEpiRowAffine.
constexpr int kEpiFoldA = 5;
constexpr int kEpiFoldAGelu = 6;
constexpr int kEpiFoldCStats = 7;

// GELU(x) = 0.5 x (1 + erf(x / sqrt 2)) = max(x, 0) - 0.5 |x| erfc(|x| / sqrt 2)
// (x >= 0: 1 + erf = 2 - erfc; x < 0: 1 + erf = erfc(|z|); no cancellation on
// the negative side), with erfc(a / sqrt 2) = 2^P(a): P is the degree-6 least
// squares fit of log2 erfc(a / sqrt 2) on [0, 8], weighted by the sensitivity
// of GELU to it.  Absolute error <= 2.7e-7 over fp32 inputs (the fp32 rounding
// of the result itself near |x| = 4), at most one fp16 ulp away from the
// exactly rounded value.  Beyond a = 8 the factor stays at 2^P(8) ~ 1e-15.
// Six FMAs and one exp2: the epilogue runs when no MFMA work is left to hide
// it, so its instruction count is wall time; the library erff costs 3x this.
__device__ __forceinline__ float geluErf(float x) {
  const float ax = fabsf(x);
  const float a = fminf(ax, 8.0f);
  float P = fmaf(3.448796997e-05f, a, -7.812886615e-04f);
  P = fmaf(P, a, 8.119936101e-03f);
  P = fmaf(P, a, -5.347220227e-02f);
  P = fmaf(P, a, -4.587264359e-01f);
  P = fmaf(P, a, -1.151216269e+00f);
  P = fmaf(P, a, 8.451195754e-06f);
  return fmaf(-0.5f * ax, __builtin_amdgcn_exp2f(P), fmaxf(x, 0.0f));
}
// 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3)
__device__ __forceinline__ float geluTanh(float x) {
  // exp(-2u) = exp2(-2 log2(e) u) = exp2(x (c1 + c3 x^2)) with the constants
  // folded: c1 = -2 log2(e) sqrt(2/pi), c3 = 0.044715 c1 (three multiplies
  // fewer per output; the epilogue's instruction count is wall time).
  // Large negative x gives x * rcp(inf) = -0.
  const float w = fmaf(x * x, -0.1029432397f, -2.3022081983f);
  const float e = __builtin_amdgcn_exp2f(x * w);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

template <int EPI> __device__ __forceinline__ float activate(float v) {
  if (EPI == int(Epilogue::kGeluErf))
    return geluErf(v);
  if (EPI == int(Epilogue::kGeluTanh))
    return geluTanh(v);
  return v;
}

// XCD-contiguous tile id for this workgroup.
__device__ __forceinline__ int tileForBlock(int nTiles, int pid) {
  const int q = nTiles / kNumXcd, r = nTiles % kNumXcd;
  const int xcd = pid % kNumXcd, loc = pid / kNumXcd;
  return xcd * q + (xcd < r ? xcd : r) + loc;
}

// Tile id -> (tile row, tile column).  Ids walk groups of kGroupM tile rows
// column by column, so that the workgroups running at the same time on one XCD
// cover a compact block of D and share both A rows and B columns in that XCD's
// L2 instead of streaming all of B for every tile row.
constexpr int kGroupM = 8;
__device__ __forceinline__ void tileCoords(int tile, int tilesM, int tilesN,
                                           int *tileM, int *tileN) {
  const int groupSize = kGroupM * tilesN;
  const int g = tile / groupSize;
  const int firstM = g * kGroupM;
  const int rows = tilesM - firstM < kGroupM ? tilesM - firstM : kGroupM;
  const int inGroup = tile - g * groupSize;
  *tileM = firstM + inGroup % rows;
  *tileN = inGroup / rows;
}

// n / d for n < 2^32 given m = floor(2^32 / d) (0xffffffff for d == 1): the
// high product is the quotient or one less.
__device__ __forceinline__ uint32_t divByMagic(uint32_t n, uint32_t d,
                                               uint32_t m) {
  const uint32_t q = __umulhi(n, m);
  return n - q * d >= d ? q + 1 : q;
}
inline uint32_t magicFor(uint32_t d) {
  return d <= 1 ? 0xffffffffu : uint32_t((uint64_t(1) << 32) / d);
}

// m % cRowPeriod (the row of a shared source that output row m reads).
__device__ __forceinline__ int rowInPeriod(const GemmParams &p, int m) {
  const uint32_t q =
      divByMagic(uint32_t(m), uint32_t(p.cRowPeriod), p.cRowMagic);
  return m - int(q) * p.cRowPeriod;
}

// tileForBlock + tileCoords with the divisions prepared on the host; returns
// the tile id (what tileCoords maps to the same coordinates).
__device__ __forceinline__ int tileCoordsFast(const GemmParams &p, int pid,
                                              int *tileM, int *tileN) {
  const int xcd = pid & (kNumXcd - 1), loc = pid >> 3;
  static_assert(kNumXcd == 8, "pid >> 3");
  const uint32_t tile =
      uint32_t(xcd * p.xcdQ + (xcd < p.xcdR ? xcd : p.xcdR) + loc);
  const uint32_t groupSize = uint32_t(kGroupM * p.tilesN);
  const uint32_t g = divByMagic(tile, groupSize, p.groupMagic);
  const uint32_t inGroup = tile - g * groupSize;
  static_assert(kGroupM == 8, "inGroup >> 3");
  if (int(g) < p.fullGroups) {
    *tileM = int(g * kGroupM + (inGroup & (kGroupM - 1)));
    *tileN = int(inGroup >> 3);
  } else {
    // (only the workgroups of a last, partial group of tile rows get here)
    const uint32_t q = inGroup / uint32_t(p.lastRows);
    *tileM = int(g * kGroupM + inGroup - q * uint32_t(p.lastRows));
    *tileN = int(q);
  }
  return int(tile);
}

// Accumulator layout shared by every kernel here (transposed 32x32 block):
// accumulator e of lane l is column 8*(e/4) + 4*(l/32) + e%4, row l%32.
template <int MI, int NI, int WTM, int WTN, int EPI, int VEC>
__device__ __forceinline__ void epilogueStore(const GemmParams &p,
                                              float16v (&acc)[MI][NI], int m0,
                                              int n0, int waveM, int waveN,
                                              int lane) {
  const int l32 = lane % 32, kb = lane / 32;
  const bool useC = p.beta != 0.f;
  // 8-byte accesses need rows of C and D that start 8-byte aligned
  const bool quadRows = p.ldd % 4 == 0 && (!useC || p.ldc % 4 == 0);
#pragma unroll
  for (int i = 0; i < MI; i++) {
    const int m = m0 + waveM * WTM + i * 32 + l32;
    if (m >= p.M)
      continue;
    const int64_t cRow = int64_t(rowInPeriod(p, m)) * p.ldc;
    const int64_t dRow = int64_t(m) * p.ldd;
#pragma unroll
    for (int j = 0; j < NI; j++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int n = n0 + waveN * WTN + j * 32 + g * 8 + kb * 4;
        if (VEC == 8 && quadRows && n + 4 <= p.N) {
          float c[4] = {0.f, 0.f, 0.f, 0.f};
          if (useC) {
            const half4 cv = *reinterpret_cast<const half4 *>(p.C + cRow + n);
#pragma unroll
            for (int e = 0; e < 4; e++)
              c[e] = float(cv[e]);
          }
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            float v = p.alpha * acc[i][j][g * 4 + e];
            if (useC)
              v += p.beta * c[e];
            o[e] = _Float16(activate<EPI>(v));
          }
          *reinterpret_cast<half4 *>(p.D + dRow + n) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (n + e < p.N) {
              float v = p.alpha * acc[i][j][g * 4 + e];
              if (useC)
                v += p.beta * float(p.C[cRow + n + e]);
              p.D[dRow + n + e] = _Float16(activate<EPI>(v));
            }
          }
        }
      }
    }
  }
}

// Same result as epilogueStore for 8-aligned problems, with full-width memory
// accesses: each wavefront turns its accumulators around through a private LDS
// strip (32 rows x WTN fp32, rows padded by 16 bytes), so that a lane ends up
// with 8 consecutive columns of one row and reads C / writes D 16 bytes at a
// time, a row segment of WTN halves per WTN/8 lanes.  In accumulator order a
// store instruction scatters 16-byte pieces over 32 rows, which costs more
// than a microsecond on a 1024 x 3072 output.  `smem` is the main loop's LDS;
// the barrier makes sure no wavefront still reads operands from it.
template <int MI, int NI, int WTM, int WTN, int EPI>
__device__ __forceinline__ void
epilogueStoreLds(const GemmParams &p, float16v (&acc)[MI][NI], int m0, int n0,
                 int waveM, int waveN, int lane, int wave,
                 unsigned char *smem) {
  constexpr int ROW_B = WTN * 4 + 16;
  constexpr int LPR = WTN / 8;  // lanes per row on the way out
  constexpr int RPP = 64 / LPR; // rows per pass
  // a row width that does not divide the wavefront (96 columns: 12 lanes per
  // row) leaves 64 - RPP * LPR lanes without work and a partial last pass
  constexpr int PASSES = (32 + RPP - 1) / RPP;
  constexpr bool kEven = RPP * LPR == 64 && PASSES * RPP == 32;
  unsigned char *mine = smem + wave * (32 * ROW_B);
  const int l32 = lane % 32, kb = lane / 32;
  const bool useC = p.beta != 0.f;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
  const bool laneActive = kEven || lane < RPP * LPR;
  const int n = n0 + waveN * WTN + cc;
  // 16-byte accesses need rows of C and D that start 16-byte aligned
  const bool vec16 = p.ldd % 8 == 0 && (!useC || p.ldc % 8 == 0);
  // Row-affine kernels: column sums of B for this lane's 8 columns (the same
  // columns in every pass), summed over the slices they were computed in.
  float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if constexpr (EPI == kEpiRowAffine) {
    if (n < p.N)
      for (int sl = 0; sl < p.colSumSlices; sl++) {
        const float4v *src = reinterpret_cast<const float4v *>(
            p.colSum + int64_t(sl) * p.N + n);
        const float4v a = src[0], b = src[1];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          cs[e] += a[e];
          cs[e + 4] += b[e];
        }
      }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MI; i++) {
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        float4v v;
#pragma unroll
        for (int e = 0; e < 4; e++)
          v[e] = acc[i][j][g * 4 + e];
        *reinterpret_cast<float4v *>(mine + l32 * ROW_B +
                                     (j * 32 + g * 8 + kb * 4) * 4) = v;
      }
#pragma unroll
    for (int pass = 0; pass < PASSES; pass++) {
      const int rWant = pass * RPP + rr;
      const bool rowActive = laneActive && (kEven || rWant < 32);
      const int r = kEven ? rWant : (rWant < 32 ? rWant : 31);
      const float4v lo =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4);
      const float4v hi =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4 + 16);
      const int m = m0 + waveM * WTM + i * 32 + r;
      float rowSum = 0.f, rowSq = 0.f;
      if (rowActive && m < p.M && n < p.N) {
        const _Float16 *cPtr = p.C + int64_t(rowInPeriod(p, m)) * p.ldc + n;
        _Float16 *dPtr = p.D + int64_t(m) * p.ldd + n;
        float c[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (useC) {
          if (vec16) {
            const half8 cv = *reinterpret_cast<const half8 *>(cPtr);
#pragma unroll
            for (int e = 0; e < 8; e++)
              c[e] = float(cv[e]);
          } else {
            // rows start at 4-byte boundaries only (N not a multiple of 8):
            // pairs, and the pair that reaches past column N is dropped (N even)
#pragma unroll
            for (int e = 0; e < 8; e += 2)
              if (n + e < p.N) {
                const half2v cv = *reinterpret_cast<const half2v *>(cPtr + e);
                c[e] = float(cv[0]);
                c[e + 1] = float(cv[1]);
              }
          }
        }
        float rowScale = 1.f, rowShift = 0.f;
        if constexpr (EPI == kEpiRowAffine) {
          rowScale = float(p.rowScale[m]);
          rowShift = float(p.rowShift[m]);
        }
        half8 o;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          float a = e < 4 ? lo[e] : hi[e - 4];
          if constexpr (EPI == kEpiRowAffine)
            a = fmaf(rowScale, a, rowShift * cs[e]);
          float v = p.alpha * a;
          if (useC)
            v += p.beta * c[e];
          o[e] = _Float16(activate<EPI>(v));
        }
        if constexpr (EPI == kEpiRowStats) {
          // statistics of the values as stored
#pragma unroll
          for (int e = 0; e < 8; e++)
            if (n + e < p.N) {
              const float x = float(o[e]);
              rowSum += x;
              rowSq = fmaf(x, x, rowSq);
            }
        }
        if (vec16) {
          storeWriteThrough(reinterpret_cast<half8 *>(dPtr), o);
        } else if (n + 8 <= p.N) {
          // rows start at 4-byte boundaries only (N even, not a multiple of 8):
          // still one 16-byte store, which the hardware takes at dword
          // alignment (as it does the 16-byte loads of such a B); written as
          // asm because a C++ store of this type would promise 16-byte
          // alignment.  Default cache policy: see store_policy.h.
          typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
          asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1"
                       :
                       : "v"(dPtr), "v"(__builtin_bit_cast(u32x4, o))
                       : "memory");
        } else {
          // the row's last vector: pairs, the pair past column N is dropped
#pragma unroll
          for (int e = 0; e < 8; e += 2)
            if (n + e < p.N) {
              half2v ov;
              ov[0] = o[e];
              ov[1] = o[e + 1];
              *reinterpret_cast<half2v *>(dPtr + e) = ov;
            }
        }
      }
      if constexpr (EPI == kEpiRowStats) {
        static_assert(EPI != kEpiRowStats || kEven,
                      "row statistics need a power-of-two wave tile width");
        // the LPR lanes of a row hold its WTN columns: one partial per row and
        // wavefront column
        rowSum = sumAcrossLanes<LPR>(rowSum);
        rowSq = sumAcrossLanes<LPR>(rowSq);
        if (lane % LPR == 0 && m < p.M) {
          const int piece = (n0 + waveN * WTN) / WTN;
          float2v st;
          st[0] = rowSum;
          st[1] = rowSq;
          *reinterpret_cast<float2v *>(p.rowStatPartials +
                                       (int64_t(piece) * p.M + m) * 2) = st;
        }
      }
    }
  }
}

// The same result as epilogueStoreLds for the common cases, without its
// per-row address arithmetic and branches: N, ldd (and ldc) multiples of 8 with
// 16-byte aligned C / D, and a source that is absent, one bias row, or a full
// [M, N] matrix (epilogueFastFits).  Accumulators go through the wavefront's
// private LDS strip as in epilogueStoreLds; C and D are addressed through
// buffer descriptors based at the wavefront's first row (rows past M fall
// outside the descriptor and are dropped by the hardware, columns past N get
// an out-of-range offset); the source vectors of every pass are requested
// before the transposition starts.  On a 1024 x 3072 output this takes 0.6 us
// off the bias + GELU epilogue and 0.9 us off the residual one.
// CMODE: 0 no source, 1 one bias row, 2 full [M, N] matrix.
template <int MI, int NI, int WTM, int WTN, int EPI, int CMODE>
__device__ __forceinline__ void
epilogueFast(const GemmParams &p, float16v (&acc)[MI][NI], int m0, int n0,
             int waveM, int waveN, int lane, int wave, unsigned char *smem) {
  constexpr int ROW_B = WTN * 4 + 16;
  constexpr int LPR = WTN / 8;  // lanes per row on the way out
  constexpr int RPP = 64 / LPR; // rows per pass
  // a row width that does not divide the wavefront (96 columns: 12 lanes per
  // row) leaves 64 - RPP * LPR lanes without work and a partial last pass;
  // those lanes and rows get an offset outside the descriptors
  constexpr int PASSES = (32 + RPP - 1) / RPP;
  constexpr bool kEven = RPP * LPR == 64 && PASSES * RPP == 32;
  constexpr uint32_t kOob = 0x80000000u;
  unsigned char *mine = smem + wave * (32 * ROW_B);
  const int l32 = lane % 32, kb = lane / 32;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
  const bool laneActive = kEven || lane < RPP * LPR;
  const int rowBase = m0 + waveM * WTM;
  const int colBase = n0 + waveN * WTN;
  const int n = colBase + cc;
  auto clampBytes = [](int64_t b) -> int32_t {
    return b > 0x7fffffffLL ? 0x7fffffff : (b < 0 ? 0 : int32_t(b));
  };
  const int rowsLeft = p.M - rowBase;
  const auto rsrcD = __builtin_amdgcn_make_buffer_rsrc(
      p.D + int64_t(rowBase) * p.ldd + colBase, 0,
      clampBytes((int64_t(rowsLeft) * p.ldd - colBase) * 2), 0x00020000);
  const uint32_t ldd2 = uint32_t(p.ldd) * 2u, ldc2 = uint32_t(p.ldc) * 2u;
  const uint32_t colOff = n < p.N && laneActive ? uint32_t(cc) * 2u : kOob;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  // source vectors
  float bias[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  half8 cv[MI][PASSES];
  if constexpr (CMODE == 1) {
    if (n < p.N) {
      const half8 b = *reinterpret_cast<const half8 *>(p.C + n);
#pragma unroll
      for (int e = 0; e < 8; e++)
        bias[e] = float(b[e]);
    }
  } else if constexpr (CMODE == 2) {
    const auto rsrcC = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(p.C) + int64_t(rowBase) * p.ldc + colBase, 0,
        clampBytes((int64_t(rowsLeft) * p.ldc - colBase) * 2), 0x00020000);
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int ps = 0; ps < PASSES; ps++) {
        const uint32_t r = uint32_t(i * 32 + ps * RPP + rr);
        const bool off = colOff == kOob || (!kEven && ps * RPP + rr >= 32);
        cv[i][ps] = __builtin_bit_cast(
            half8, __builtin_amdgcn_raw_buffer_load_b128(
                       rsrcC, off ? kOob : r * ldc2 + colOff, 0, 0));
      }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MI; i++) {
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        float4v v;
#pragma unroll
        for (int e = 0; e < 4; e++)
          v[e] = acc[i][j][g * 4 + e];
        *reinterpret_cast<float4v *>(mine + l32 * ROW_B +
                                     (j * 32 + g * 8 + kb * 4) * 4) = v;
      }
#pragma unroll
    for (int ps = 0; ps < PASSES; ps++) {
      const int rWant = ps * RPP + rr;
      const bool off = colOff == kOob || (!kEven && rWant >= 32);
      const int r = kEven ? rWant : (rWant < 32 ? rWant : 31);
      const float4v lo =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4);
      const float4v hi =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4 + 16);
      half8 o;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float v = p.alpha * (e < 4 ? lo[e] : hi[e - 4]);
        if constexpr (CMODE == 1)
          v = fmaf(p.beta, bias[e], v);
        if constexpr (CMODE == 2)
          v = fmaf(p.beta, float(cv[i][ps][e]), v);
        o[e] = _Float16(activate<EPI>(v));
      }
      const uint32_t row = uint32_t(i * 32 + r);
      __builtin_amdgcn_raw_buffer_store_b128(
          __builtin_bit_cast(u32x4, o), rsrcD,
          off ? kOob : row * ldd2 + colOff, 0, kWriteThroughAux);
    }
  }
}


// (rstd, -mean * rstd) of row m0 + tid of a folded layer norm, for the first BM
// threads of the workgroup, in two steps: foldRowStatRequest asks for the
// row's first pieces (no branch around a load: an index past the last piece
// re-reads the last piece, so the batch is one memory round trip) and
// foldRowStatFinish adds them up (pieces beyond the batch, which no BERT shape
// has, are fetched there).  The kernels request next to their first slab loads; the
// round trip then overlaps the main loop (tiles with registers to spare keep
// those pairs until the epilogue) or the wait for the first slab (256-row
// tiles finish at once).  kFoldBatch: pieces requested up front, sized for rows
// of up to 1024 columns (BERT's hidden sizes) cut into tiles BM wide.
template <int BM> struct FoldBatch {
  static constexpr int value = BM >= 256 ? 4 : (BM >= 128 ? 8 : 16);
};
template <int BM>
__device__ __forceinline__ void
foldRowStatRequest(const GemmParams &p, int m0, int tid,
                   float2v (&v)[FoldBatch<BM>::value]) {
  constexpr int kFoldBatch = FoldBatch<BM>::value;
  // Every thread loads, from an address that is always valid, so that nothing
  // stands between these requests and the ones around them: threads past the
  // tile's rows repeat a row, and without statistics the first bytes of A's
  // rows are read (and ignored by foldRowStatFinish).
  const bool folded = p.foldStats != nullptr;
  const float *base =
      folded ? p.foldStats : reinterpret_cast<const float *>(p.A);
  const int pieces = folded ? p.foldPieces : 1;
  const int row = m0 + (tid < BM ? tid : 0);
  const int m = row < p.M ? row : p.M - 1;
#pragma unroll
  for (int u = 0; u < kFoldBatch; u++) {
    const int at = u < pieces ? u : pieces - 1;
    v[u] = *reinterpret_cast<const float2v *>(base +
                                              (int64_t(at) * p.M + m) * 2);
  }
}
template <int BM>
__device__ __forceinline__ float2v
foldRowStatFinish(const GemmParams &p, int m0, int tid,
                  const float2v (&v)[FoldBatch<BM>::value]) {
  constexpr int kFoldBatch = FoldBatch<BM>::value;
  float2v stat{1.f, 0.f};
  if (p.foldStats != nullptr && tid < BM) {
    const int m = m0 + tid < p.M ? m0 + tid : p.M - 1;
    float s = 0.f, sq = 0.f;
#pragma unroll
    for (int u = 0; u < kFoldBatch; u++) {
      s += u < p.foldPieces ? v[u][0] : 0.f;
      sq += u < p.foldPieces ? v[u][1] : 0.f;
    }
    for (int pc = kFoldBatch; pc < p.foldPieces; pc++) {
      const float2v w = *reinterpret_cast<const float2v *>(
          p.foldStats + (int64_t(pc) * p.M + m) * 2);
      s += w[0];
      sq += w[1];
    }
    const float mu = s * p.foldInvN;
    // the difference cancels to a small negative number for near-constant
    // rows; clamped so that a tiny eps cannot turn it into a NaN
    const float rstd =
        1.0f / sqrtf(fmaxf(sq * p.foldInvN - mu * mu, 0.f) + p.foldEps);
    stat[0] = rstd;
    stat[1] = -mu * rstd;
  }
  return stat;
}

// The epilogues with a folded layer norm (kEpiFold*).  Same memory access
// scheme as epilogueFast (buffer descriptors per wavefront, 16-byte accesses,
// every source vector requested before the transposition): N, ldd and ldc
// multiples of 8, C / D 16-byte aligned, C absent or a full [M, N] matrix; the
// host checks this.  myStat: foldRowStat() of this thread's row; the pairs of
// the workgroup's BM rows meet in LDS, behind the wavefronts' accumulator
// strips.
template <int MI, int NI, int WTM, int WTN, int EPI, int BM, int THREADS>
__device__ __forceinline__ void
epilogueFold(const GemmParams &p, float16v (&acc)[MI][NI], int m0, int n0,
             int waveM, int waveN, int lane, int wave, int tid,
             float2v myStat, unsigned char *smem) {
  constexpr bool kFoldA = EPI == kEpiFoldA || EPI == kEpiFoldAGelu;
  constexpr bool kFoldC = EPI == kEpiFoldCStats;
  constexpr bool kStats = EPI == kEpiFoldCStats;
  constexpr int ROW_B = WTN * 4 + 16;
  constexpr int LPR = WTN / 8;  // lanes per row on the way out
  constexpr int RPP = 64 / LPR; // rows per pass
  constexpr int PASSES = 32 / RPP;
  static_assert(RPP * LPR == 64 && PASSES * RPP == 32,
                "folded epilogues need a power-of-two wave tile width");
  constexpr uint32_t kOob = 0x80000000u;
  constexpr int kStripBytes = (THREADS / kWave) * 32 * ROW_B;
  constexpr int WN_ = (THREADS / kWave) / (BM / WTM); // wavefront columns
  unsigned char *mine = smem + wave * (32 * ROW_B);
  float2v *rowStat = reinterpret_cast<float2v *>(smem + kStripBytes);
  // (kStats) partial sums of the tile's rows per wavefront column, [BM][WN]
  float2v *tileSums = rowStat + BM;
  const int l32 = lane % 32, kb = lane / 32;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
  const int rowBase = m0 + waveM * WTM;
  const int colBase = n0 + waveN * WTN;
  const int n = colBase + cc;
  auto clampBytes = [](int64_t b) -> int32_t {
    return b > 0x7fffffffLL ? 0x7fffffff : (b < 0 ? 0 : int32_t(b));
  };
  const int rowsLeft = p.M - rowBase;
  const auto rsrcD = __builtin_amdgcn_make_buffer_rsrc(
      p.D + int64_t(rowBase) * p.ldd + colBase, 0,
      clampBytes((int64_t(rowsLeft) * p.ldd - colBase) * 2), 0x00020000);
  const uint32_t ldd2 = uint32_t(p.ldd) * 2u, ldc2 = uint32_t(p.ldc) * 2u;
  const uint32_t colOff = n < p.N ? uint32_t(cc) * 2u : kOob;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  const bool useC = p.beta != 0.f;
  const bool folded = p.foldStats != nullptr;
  // column sums of B for this lane's 8 columns (the same in every pass)
  float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if constexpr (kFoldA) {
    if (folded && n < p.N) {
      const float4v *src = reinterpret_cast<const float4v *>(p.colSum + n);
      const float4v a = src[0], b = src[1];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        cs[e] = a[e];
        cs[e + 4] = b[e];
      }
    }
  }
  half8 cv[MI][PASSES];
  if (useC) {
    const auto rsrcC = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(p.C) + int64_t(rowBase) * p.ldc + colBase, 0,
        clampBytes((int64_t(rowsLeft) * p.ldc - colBase) * 2), 0x00020000);
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int ps = 0; ps < PASSES; ps++) {
        const uint32_t r = uint32_t(i * 32 + ps * RPP + rr);
        cv[i][ps] = __builtin_bit_cast(
            half8, __builtin_amdgcn_raw_buffer_load_b128(
                       rsrcC, colOff == kOob ? kOob : r * ldc2 + colOff, 0, 0));
      }
  }
  __syncthreads(); // no wavefront still reads operands from the main loop's LDS
  if (tid < BM)
    rowStat[tid] = myStat;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MI; i++) {
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        float4v v;
#pragma unroll
        for (int e = 0; e < 4; e++)
          v[e] = acc[i][j][g * 4 + e];
        *reinterpret_cast<float4v *>(mine + l32 * ROW_B +
                                     (j * 32 + g * 8 + kb * 4) * 4) = v;
      }
#pragma unroll
    for (int ps = 0; ps < PASSES; ps++) {
      const int r = ps * RPP + rr;
      const float4v lo =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4);
      const float4v hi =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4 + 16);
      const float2v st = rowStat[waveM * WTM + i * 32 + r];
      half8 o;
      float rowSum = 0.f, rowSq = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float a = e < 4 ? lo[e] : hi[e - 4];
        if constexpr (kFoldA)
          a = fmaf(st[0], a, st[1] * cs[e]);
        float v = p.alpha * a;
        if (useC) {
          float c = float(cv[i][ps][e]);
          if constexpr (kFoldC)
            c = fmaf(c, st[0], st[1]);
          v = fmaf(p.beta, c, v);
        }
        if constexpr (EPI == kEpiFoldAGelu)
          v = geluErf(v);
        o[e] = _Float16(v);
        if constexpr (kStats) {
          // statistics of the values as stored
          const float x = float(o[e]);
          rowSum += x;
          rowSq = fmaf(x, x, rowSq);
        }
      }
      const uint32_t row = uint32_t(i * 32 + r);
      __builtin_amdgcn_raw_buffer_store_b128(
          __builtin_bit_cast(u32x4, o), rsrcD,
          colOff == kOob ? kOob : row * ldd2 + colOff, 0, kWriteThroughAux);
      if constexpr (kStats) {
        // the LPR lanes of a row hold its WTN columns (columns past N
        // contribute nothing); the wavefront columns of the tile meet in LDS
        if (colOff == kOob)
          rowSum = rowSq = 0.f;
        rowSum = sumAcrossLanes<LPR>(rowSum);
        rowSq = sumAcrossLanes<LPR>(rowSq);
        if (lane % LPR == 0) {
          float2v out;
          out[0] = rowSum;
          out[1] = rowSq;
          tileSums[(waveM * WTM + int(row)) * WN_ + waveN] = out;
        }
      }
    }
  }
  if constexpr (kStats) {
    // one (sum, sum of squares) pair per row and tile column: piece n0 / BN
    __syncthreads();
    if (tid < BM && m0 + tid < p.M) {
      float2v out{0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WN_; w++) {
        out[0] += tileSums[tid * WN_ + w][0];
        out[1] += tileSums[tid * WN_ + w][1];
      }
      const int piece = n0 / (WTN * WN_);
      // (written through: the next kernel reads them first thing)
      storeWriteThrough(reinterpret_cast<float2v *>(
                            p.rowStatPartials +
                            (int64_t(piece) * p.M + m0 + tid) * 2),
                        out);
    }
  }
}

// Whether epilogueFast applies (wave-uniform), and with which source mode
// (0 none, 1 bias row, 2 full matrix); -1 = use epilogueStoreLds.
__host__ __device__ __forceinline__ int epilogueFastMode(const GemmParams &p,
                                                         int tileM) {
  auto al16 = [](const void *q) {
    return (reinterpret_cast<uintptr_t>(q) & 15) == 0;
  };
  // 32-bit byte offsets inside a wavefront's rows
  if (p.N % 8 != 0 || p.ldd % 8 != 0 || !al16(p.D) ||
      int64_t(tileM) * p.ldd * 2 >= (int64_t(1) << 31))
    return -1;
  if (p.beta == 0.f)
    return 0;
  if (!al16(p.C))
    return -1;
  if (p.cRowPeriod == 1)
    return 1;
  if (p.cRowPeriod >= p.M && p.ldc % 8 == 0 &&
      int64_t(tileM) * p.ldc * 2 < (int64_t(1) << 31))
    return 2;
  return -1;
}

// Dispatch: the fast epilogue where it applies, the general one otherwise.
template <int MI, int NI, int WTM, int WTN, int EPI>
__device__ __forceinline__ void
epilogueAuto(const GemmParams &p, float16v (&acc)[MI][NI], int m0, int n0,
             int waveM, int waveN, int lane, int wave, unsigned char *smem) {
  static_assert(EPI < kEpiFoldA, "folded epilogues are called directly");
  if constexpr (EPI <= int(Epilogue::kGeluTanh)) {
    const int mode = p.epiMode;
    if (mode == 0)
      return epilogueFast<MI, NI, WTM, WTN, EPI, 0>(p, acc, m0, n0, waveM, waveN,
                                                    lane, wave, smem);
    if (mode == 1)
      return epilogueFast<MI, NI, WTM, WTN, EPI, 1>(p, acc, m0, n0, waveM, waveN,
                                                    lane, wave, smem);
    if (mode == 2)
      return epilogueFast<MI, NI, WTM, WTN, EPI, 2>(p, acc, m0, n0, waveM, waveN,
                                                    lane, wave, smem);
  }
  epilogueStoreLds<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane,
                                          wave, smem);
}

// Partial tile of one K slice -> workspace, in accumulator order (coalesced
// 128-bit stores; the reduce kernel uses the same thread -> element mapping).
template <int MI, int NI, int THREADS>
__device__ __forceinline__ void storePartial(const GemmParams &p,
                                             float16v (&acc)[MI][NI], int tile,
                                             int slice, int numSlices,
                                             int tid) {
  constexpr int ACC_V4 = MI * NI * 4;
  float4v *mine = reinterpret_cast<float4v *>(p.workspace) +
                  (int64_t(tile) * numSlices + slice) * (ACC_V4 * THREADS);
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        float4v v;
#pragma unroll
        for (int e = 0; e < 4; e++)
          v[e] = acc[i][j][g * 4 + e];
        mine[((i * NI + j) * 4 + g) * THREADS + tid] = v;
      }
}

// In-kernel form of the split-K reduction, first half: this workgroup's
// partial tile is in the workspace; count it in the tile's arrival word and
// tell whether it was the last of the tile's slices to get there.  The last
// one sums all the partial tiles (sumPartials) and finishes the tile; the
// others are done with it.  No workgroup ever waits for another.
//
// All slices of a tile run on one XCD (the launcher's condition), so they
// share an L2.  A slice's stores are in that L2 once its vmcnt has drained
// (the vector L1 writes through); the barrier extends that to the workgroup,
// and the atomic that follows goes to the same L2.  The last arriver drops its
// L1 (buffer_inv sc0) so that its loads come from the L2 -- the lines could
// only be in its L1 by accident of an earlier tile, but an accident is enough.
// The arrival word also counts the slices per XCD (seven bits each above the
// eight-bit total): a last arriver that does not find every slice on its own
// XCD raises the host-visible flag, the library's check that the placement it
// relies on held.  The word goes back to zero for the next launch.
// `lds` is any four bytes of LDS nobody else uses between the two barriers.
__device__ __forceinline__ bool arriveAtTile(const GemmParams &p, int tile,
                                             int numSlices, int tid,
                                             void *lds) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  volatile uint32_t *wasLast = static_cast<volatile uint32_t *>(lds);
  if (tid == 0) {
    uint32_t xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    xcc &= 7u;
    const unsigned long long mine = 1ull | (1ull << (8 + 7 * xcc));
    const unsigned long long seen =
        __hip_atomic_fetch_add(&p.tileArrivals[tile], mine, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT) +
        mine;
    const bool last = uint32_t(seen & 255u) == uint32_t(numSlices);
    if (last) {
      if (uint32_t((seen >> (8 + 7 * xcc)) & 127u) != uint32_t(numSlices))
        __hip_atomic_store(p.misplaced, 1u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(&p.tileArrivals[tile], 0ull, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    *wasLast = last ? 1u : 0u;
  }
  __syncthreads();
  const bool last = __builtin_amdgcn_readfirstlane(int(*wasLast)) != 0;
  __syncthreads(); // the epilogue's strips may overwrite that word
  if (last)
    asm volatile("buffer_inv sc0\n\ts_waitcnt vmcnt(0)" ::: "memory");
  return last;
}

// Second half: the tile's partial tiles, added in slice order starting from
// zero -- the sum splitKReduceKernel forms, bit for bit.
template <int MI, int NI, int THREADS>
__device__ __forceinline__ void sumPartials(const GemmParams &p,
                                            float16v (&acc)[MI][NI], int tile,
                                            int numSlices, int tid) {
  constexpr int ACC_V4 = MI * NI * 4;
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[i][j][e] = 0.f;
  const float4v *part = reinterpret_cast<const float4v *>(p.workspace) +
                        int64_t(tile) * numSlices * (ACC_V4 * THREADS) + tid;
  // Loads of up to AHEAD slices are in flight before the first add: one
  // workgroup walks all the slices, and a small tile has only a few loads per
  // slice to hide the L2's latency behind.
  constexpr int AHEAD = ACC_V4 <= 4 ? 4 : ACC_V4 <= 8 ? 2 : 1;
  int s = 0;
  if constexpr (AHEAD > 1) {
    for (; s + AHEAD <= numSlices; s += AHEAD, part += AHEAD * ACC_V4 * THREADS) {
      float4v v[AHEAD][ACC_V4];
#pragma unroll
      for (int u = 0; u < AHEAD; u++)
#pragma unroll
        for (int q = 0; q < ACC_V4; q++)
          v[u][q] = part[(u * ACC_V4 + q) * THREADS];
#pragma unroll
      for (int u = 0; u < AHEAD; u++) // slice order
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
          for (int j = 0; j < NI; j++)
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
              for (int e = 0; e < 4; e++)
                acc[i][j][g * 4 + e] += v[u][(i * NI + j) * 4 + g][e];
    }
  }
  for (; s < numSlices; s++, part += ACC_V4 * THREADS) {
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int j = 0; j < NI; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const float4v v = part[((i * NI + j) * 4 + g) * THREADS];
#pragma unroll
          for (int e = 0; e < 4; e++)
            acc[i][j][g * 4 + e] += v[e];
        }
  }
}

template <int BM, int BN, int WM, int WN, int EPI, int VEC>
__global__ __launch_bounds__(WM *WN *kWave) void splitKReduceKernel(
    GemmParams p, int numSlices) {
  constexpr int THREADS = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int ACC_V4 = MI * NI * 4;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int tile = blockIdx.x;
  int tileM, tileN;
  tileCoords(tile, p.tilesM, p.tilesN, &tileM, &tileN);
  float16v acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[i][j][e] = 0.f;
  const float4v *ws = reinterpret_cast<const float4v *>(p.workspace) +
                      int64_t(tile) * numSlices * (ACC_V4 * THREADS);
  for (int s = 0; s < numSlices; s++) {
    const float4v *part = ws + int64_t(s) * (ACC_V4 * THREADS);
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int j = 0; j < NI; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const float4v v = part[((i * NI + j) * 4 + g) * THREADS + tid];
#pragma unroll
          for (int e = 0; e < 4; e++)
            acc[i][j][g * 4 + e] += v[e];
        }
  }
  epilogueStore<MI, NI, WTM, WTN, EPI, VEC>(p, acc, tileM * BM, tileN * BN,
                                            wave / WN, wave % WN, lane);
}

// The same reduction with one thread per group of four outputs instead of one
// workgroup per tile: a skinny problem (64 x 1024 in 16 tiles) would otherwise
// reduce on 16 workgroups, each walking the slices of a whole tile in turn.
// Thread idx owns float4 number idx of the partial-tile layout (tile, block
// row i, block column j, quad g, thread of the producing workgroup); it adds
// the slices in slice order, four loads in flight, and finishes its four
// consecutive columns of one output row.
template <int BM, int BN, int WM, int WN, int EPI, int VEC>
__global__ __launch_bounds__(256) void splitKReduceFlatKernel(GemmParams p,
                                                              int numSlices) {
  constexpr int THREADS = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int ACC_V4 = MI * NI * 4;
  constexpr int PER_TILE = ACC_V4 * THREADS; // float4 per partial tile
  const int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x;
  const int64_t total = int64_t(p.tilesM) * p.tilesN * PER_TILE;
  if (idx >= total)
    return;
  const int tile = int(idx / PER_TILE);
  const int rem = int(idx % PER_TILE);
  const int q = rem / THREADS, t = rem % THREADS;
  const int i = q / (NI * 4), j = (q / 4) % NI, g = q % 4;
  const int lane = t % kWave, wave = t / kWave;
  const int l32 = lane % 32, kb = lane / 32;
  int tileM, tileN;
  tileCoords(tile, p.tilesM, p.tilesN, &tileM, &tileN);
  const float4v *part = reinterpret_cast<const float4v *>(p.workspace) +
                        int64_t(tile) * numSlices * PER_TILE + rem;
  float4v acc = {0.f, 0.f, 0.f, 0.f};
  int sl = 0;
  for (; sl + 4 <= numSlices; sl += 4) {
    float4v v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      v[u] = part[int64_t(sl + u) * PER_TILE];
#pragma unroll
    for (int u = 0; u < 4; u++) // slice order: the sum does not depend on timing
      acc += v[u];
  }
  for (; sl < numSlices; sl++)
    acc += part[int64_t(sl) * PER_TILE];
  const int m = tileM * BM + (wave / WN) * WTM + i * 32 + l32;
  const int n = tileN * BN + (wave % WN) * WTN + j * 32 + g * 8 + kb * 4;
  if (m >= p.M)
    return;
  const bool useC = p.beta != 0.f;
  const int64_t cRow = int64_t(rowInPeriod(p, m)) * p.ldc;
  const int64_t dRow = int64_t(m) * p.ldd;
  const bool quadRows = p.ldd % 4 == 0 && (!useC || p.ldc % 4 == 0);
  if (VEC == 8 && quadRows && n + 4 <= p.N) {
    float c[4] = {0.f, 0.f, 0.f, 0.f};
    if (useC) {
      const half4 cv = *reinterpret_cast<const half4 *>(p.C + cRow + n);
#pragma unroll
      for (int e = 0; e < 4; e++)
        c[e] = float(cv[e]);
    }
    half4 o;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float v = p.alpha * acc[e];
      if (useC)
        v += p.beta * c[e];
      o[e] = _Float16(activate<EPI>(v));
    }
    *reinterpret_cast<half4 *>(p.D + dRow + n) = o;
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (n + e < p.N) {
        float v = p.alpha * acc[e];
        if (useC)
          v += p.beta * float(p.C[cRow + n + e]);
        p.D[dRow + n + e] = _Float16(activate<EPI>(v));
      }
    }
  }
}

// ===================================================================== dma ==
// Swizzles (in units of 16-byte chunks / 64-byte groups inside an LDS row).
// K-contiguous tiles (A, and B given as [N, K]): rows of 128 bytes = 8 chunks;
// chunk c of row r lives at position c ^ ((r >> 1) & 7), which makes the
// 128-bit fragment reads of 16 consecutive rows hit 16 distinct bank groups.
__device__ __forceinline__ int swzK(int row, int chunk) {
  return chunk ^ ((row >> 1) & 7);
}
// Row-major B tiles: a transposing read touches rows k..k+3 and k+8..k+11, 64
// bytes of each; 64-byte group g of row k lives at position g ^ f(k).
// A 96-column tile (rows of 192 bytes, three groups) needs none: rows k..k+3
// start 192 bytes apart, which already spreads their groups over the banks.
template <int BN> __device__ __forceinline__ int swzN(int k, int group) {
  if (BN == 96)
    return group;
  if (BN == 64)
    return group ^ ((k >> 1) & 1);
  return group ^ (k & 3);
}

// ------------------------------------------------------------ kernel table --
struct LaunchPlan {
  GemmParams p;
  int splitK;
  int64_t nTiles;
  bool callerWorkspace; // partial tiles go to a buffer the caller brought
};

template <int BM, int BN, int BK>
Status planLaunch(const GemmProblem &pr, LaunchPlan *plan) {
  GemmParams &p = plan->p;
  p.A = pr.A;
  p.B = pr.B;
  p.C = pr.C;
  p.D = pr.D;
  p.M = int(pr.M);
  p.N = int(pr.N);
  p.K = int(pr.K);
  p.lda = pr.lda;
  p.ldb = pr.ldb;
  p.ldc = pr.ldc;
  p.ldd = pr.ldd;
  p.cRowPeriod = int(pr.cRowPeriod > 0 ? pr.cRowPeriod : 1);
  p.alpha = pr.alpha;
  p.beta = pr.beta;
  p.rowStatPartials = pr.rowStatPartials;
  p.rowScale = pr.rowScale;
  p.rowShift = pr.rowShift;
  p.colSum = pr.colSum;
  p.colSumSlices = pr.colSumSlices;
  p.foldStats = pr.foldStats;
  p.foldPieces = pr.foldPieces;
  p.foldInvN = pr.foldInvN;
  p.foldEps = pr.foldEps;
  p.tilesM = int((pr.M + BM - 1) / BM);
  p.tilesN = int((pr.N + BN - 1) / BN);
  const int kTiles = int((pr.K + BK - 1) / BK);
  int splitK = pr.splitK < 1 ? 1 : pr.splitK;
  if (splitK > kTiles)
    splitK = kTiles > 0 ? kTiles : 1;
  p.kTilesPerSlice = (kTiles + splitK - 1) / splitK;
  if (p.kTilesPerSlice > 0) // drop slices that rounding up left empty
    splitK = (kTiles + p.kTilesPerSlice - 1) / p.kTilesPerSlice;
  if (splitK < 1)
    splitK = 1;
  plan->splitK = splitK;
  plan->nTiles = int64_t(p.tilesM) * p.tilesN;
  HOM_CHECK_RET(plan->nTiles < (int64_t(1) << 30), Status::kInvalidArgument,
                "gemm: too many output tiles (%lld)", (long long)plan->nTiles);
  p.xcdQ = int(plan->nTiles / kNumXcd);
  p.xcdR = int(plan->nTiles % kNumXcd);
  p.groupMagic = magicFor(uint32_t(kGroupM) * uint32_t(p.tilesN));
  p.fullGroups = p.tilesM / kGroupM;
  p.lastRows = p.tilesM % kGroupM > 0 ? p.tilesM % kGroupM : kGroupM;
  p.cRowMagic = magicFor(uint32_t(p.cRowPeriod));
  // (the row range a wavefront addresses with 32-bit offsets is at most BM rows)
  p.epiMode = epilogueFastMode(p, BM);
  p.workspace = nullptr;
  p.tileArrivals = nullptr;
  p.misplaced = nullptr;
  plan->callerWorkspace = pr.workspace != nullptr;
  if (splitK > 1) {
    const size_t wsBytes =
        size_t(plan->nTiles) * splitK * size_t(BM) * BN * sizeof(float);
    if (pr.workspace) {
      // caller-provided partial-tile buffer: nothing may be allocated here
      HOM_CHECK_RET(wsBytes <= pr.workspaceBytes, Status::kInvalidArgument,
                    "gemm: split-K %d of this problem needs %zu bytes of "
                    "partial tiles, the workspace holds %zu",
                    splitK, wsBytes, pr.workspaceBytes);
      p.workspace = pr.workspace;
    } else {
      p.workspace =
          static_cast<float *>(libraryScratch(kWorkspace, wsBytes, false));
      if (!p.workspace)
        return Status::kInternal;
    }
  }
  return Status::kSuccess;
}

template <typename K> Status allowLds(K kernel, int bytes, bool *done) {
  if (!*done && bytes > 48 * 1024) {
    HOM_HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    bytes),
                Status::kInternal);
  }
  *done = true;
  return Status::kSuccess;
}

template <int BM, int BN, int WM, int WN, int EPI, int VEC>
Status launchReduce(const LaunchPlan &plan, hipStream_t s) {
  // Few tiles: spread the reduction over the chip (one thread per four outputs).
  constexpr int kPerTile = (BM / 32) * (BN / 32) * 4 * kWave; // float4 per tile
  if (plan.nTiles < 128) {
    const int64_t groups = plan.nTiles * kPerTile;
    splitKReduceFlatKernel<BM, BN, WM, WN, EPI, VEC>
        <<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s>>>(
            plan.p, plan.splitK);
    HOM_HIP_RET(hipGetLastError(), Status::kInternal);
    return Status::kSuccess;
  }
  splitKReduceKernel<BM, BN, WM, WN, EPI, VEC>
      <<<dim3((unsigned)plan.nTiles), dim3(WM * WN * kWave), 0, s>>>(
          plan.p, plan.splitK);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

} // namespace gemmk
} // namespace hom
