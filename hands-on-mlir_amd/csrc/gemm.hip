// fp16 GEMM with fp32 accumulation on the gfx950 matrix cores.
//
//   D = epilogue(alpha * A.B + beta * C)
//   A [M, K] row-major; B [K, N] row-major (or [N, K] when pre-transposed);
//   C, D [M, N] row-major, D may alias C.
//
// This replaces the CUTLASS GemmUniversal instances the reference generates
// (python/gemm_generator.py:237-278, python/hom_manifest.py:503-533) and the
// cuBLASLt call behind nvteGemmF16 (include/NVGPUKernels/GemmRunner.h:404-425).
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
//    (deterministic, fp32) and runs the epilogue.  Nothing spins or fences;
//  * workgroup ids are remapped so that each of the 8 XCDs (which receive
//    consecutive ids round-robin and have private L2s) works on a contiguous
//    run of tiles.
//
// Two main-loop families
//  * "dma" kernels (the fast path, aligned problems): K is walked in 64-wide
//    slabs through an NS-deep ring of LDS buffers filled by
//    buffer_load_dwordx4 ... lds, i.e. global memory -> LDS without passing
//    through registers.  The loads of slab k+NS-1 are in flight while slab k is
//    multiplied, which is what hides HBM/L2 latency when only one or two
//    workgroups fit a CU.  Out-of-range rows/columns/k are given an offset
//    beyond the buffer descriptor's size, for which the hardware writes zeros.
//    LDS rows are not padded (the DMA writes 1 KiB contiguous per wavefront);
//    bank conflicts are avoided by permuting 16-byte chunks inside a row, which
//    costs nothing because every lane chooses its own global address.
//    A (and B when it is [N, K]) fragments are 128-bit LDS reads.  Row-major B
//    has N contiguous while an MFMA operand wants 8 consecutive k per lane:
//    those fragments are read with ds_read_b64_tr_b16, which transposes 4 k-rows
//    x 16 columns across a group of 16 lanes.
//  * "staged" kernels (any shape / alignment, and the first bring-up path):
//    global -> registers -> LDS with two LDS buffers and 32-wide slabs; row-major
//    B is interleaved into (k, k+1) half2 pairs while it is staged.
#include "cross_lane.h"
#include "kernels.h"

#include <algorithm>
#include <type_traits>
#include <utility>

namespace hom {
namespace {

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
  int M, N, K;
  int64_t lda, ldb, ldc, ldd;
  int cRowPeriod;
  float alpha, beta;
  int tilesM, tilesN;
  int kTilesPerSlice;
  // layer-norm pair (kEpiRowStats / kEpiRowAffine kernels only)
  float *rowStatPartials;
  const _Float16 *rowScale;
  const _Float16 *rowShift;
  const float *colSum;
  int colSumSlices;
};

// Epilogue codes beyond the three activations of the manifest kernels: linear
// output plus row-statistic partial sums, and linear output of a per-row
// affine transform of A folded into the accumulator.
constexpr int kEpiRowStats = 3;
constexpr int kEpiRowAffine = 4;

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
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  // exp(-2u) = exp2(-2 log2(e) u); large negative x gives x * rcp(inf) = -0
  const float e = __builtin_amdgcn_exp2f(u * -2.88539008177792681472f);
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
    const int64_t cRow = int64_t(m % p.cRowPeriod) * p.ldc;
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
  unsigned char *mine = smem + wave * (32 * ROW_B);
  const int l32 = lane % 32, kb = lane / 32;
  const bool useC = p.beta != 0.f;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
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
    for (int pass = 0; pass < 32 / RPP; pass++) {
      const int r = pass * RPP + rr;
      const float4v lo =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4);
      const float4v hi =
          *reinterpret_cast<const float4v *>(mine + r * ROW_B + cc * 4 + 16);
      const int m = m0 + waveM * WTM + i * 32 + r;
      float rowSum = 0.f, rowSq = 0.f;
      if (m < p.M && n < p.N) {
        const _Float16 *cPtr = p.C + int64_t(m % p.cRowPeriod) * p.ldc + n;
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
          *reinterpret_cast<half8 *>(dPtr) = o;
        } else {
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
template <int BN> __device__ __forceinline__ int swzN(int k, int group) {
  if (BN == 64)
    return group ^ ((k >> 1) & 1);
  return group ^ (k & 3);
}

template <int BM, int BN, int WM, int WN, int NS, int EPI, bool B_NK>
__global__ __launch_bounds__(WM *WN *kWave) void gemmDmaKernel(GemmParams p) {
  // The body uses buffer-descriptor builtins whose types exist only for the
  // GPU target; the host pass needs just the (empty) stub to launch through.
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BK = 64;
  constexpr int THREADS = WM * WN * kWave;
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_INSTR = A_BYTES / 1024, B_INSTR = B_BYTES / 1024;
  static_assert(A_INSTR % NW == 0 && B_INSTR % NW == 0,
                "tile must split evenly over the wavefronts");
  constexpr int A_PER_W = A_INSTR / NW, B_PER_W = B_INSTR / NW;
  constexpr int LOADS_PER_TILE = A_PER_W + B_PER_W; // per wavefront
  constexpr int B_ROW_BYTES = B_NK ? 128 : BN * 2;
  constexpr int B_ROWS_PER_INSTR = 1024 / B_ROW_BYTES;
  static_assert((NS - 2) * LOADS_PER_TILE < 64, "vmcnt is a 6-bit counter");

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int waveM = wave / WN, waveN = wave % WN;
  const int l32 = lane % 32, kb = lane / 32;

  const int nTiles = p.tilesM * p.tilesN;
  const int tile = tileForBlock(nTiles, blockIdx.x);
  int tileM, tileN;
  tileCoords(tile, p.tilesM, p.tilesN, &tileM, &tileN);
  const int m0 = tileM * BM, n0 = tileN * BN;
  const int slice = blockIdx.y, numSlices = gridDim.y;
  const int kTiles = (p.K + BK - 1) / BK;
  const int ktBegin = slice * p.kTilesPerSlice;
  int ktEnd = ktBegin + p.kTilesPerSlice;
  if (ktEnd > kTiles)
    ktEnd = kTiles;

  // Buffer descriptors based at this tile's first row (A) / first row or
  // column block (B), so 32-bit offsets suffice for any matrix size.  Offsets
  // at or beyond num_records read as zero.
  constexpr uint32_t kOob = 0x80000000u;
  auto clampBytes = [](int64_t b) -> int32_t {
    return b > 0x7fffffffLL ? 0x7fffffff : (b < 0 ? 0 : int32_t(b));
  };
  const _Float16 *aBase = p.A + int64_t(m0) * p.lda;
  const int64_t aBytes = (int64_t(p.M - m0) * p.lda) * 2;
  const auto rsrcA = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(aBase), 0, clampBytes(aBytes), 0x00020000);
  const _Float16 *bBase = B_NK ? p.B + int64_t(n0) * p.ldb : p.B;
  const int64_t bBytes =
      B_NK ? (int64_t(p.N - n0) * p.ldb) * 2 : (int64_t(p.K) * p.ldb) * 2;
  const auto rsrcB = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(bBase), 0, clampBytes(bBytes), 0x00020000);
  // Row-major B deeper than 2 GiB would overflow the 32-bit offset; the host
  // rejects such problems for these kernels.

  // ---- per-lane source offsets (bytes), constant over the K walk ----
  uint32_t aOff[A_PER_W];
  int aCol[A_PER_W];
#pragma unroll
  for (int i = 0; i < A_PER_W; i++) {
    const int instr = wave * A_PER_W + i;
    const int r = instr * 8 + lane / 8;
    const int c = swzK(r, lane % 8); // logical chunk stored at this position
    aCol[i] = c * 8;
    aOff[i] = (m0 + r < p.M) ? uint32_t((int64_t(r) * p.lda + c * 8) * 2) : kOob;
  }
  uint32_t bOff[B_PER_W];
  int bK[B_PER_W]; // NK: column offset in k; KN: row (k) inside the slab
#pragma unroll
  for (int i = 0; i < B_PER_W; i++) {
    const int instr = wave * B_PER_W + i;
    if (B_NK) {
      const int r = instr * 8 + lane / 8;
      const int c = swzK(r, lane % 8);
      bK[i] = c * 8;
      bOff[i] = (n0 + r < p.N) ? uint32_t((int64_t(r) * p.ldb + c * 8) * 2) : kOob;
    } else {
      constexpr int CHUNKS = B_ROW_BYTES / 16;
      const int k = instr * B_ROWS_PER_INSTR + lane / CHUNKS;
      const int pc = lane % CHUNKS; // physical chunk
      const int g = swzN<BN>(k, pc / 4);
      const int n = (g * 4 + pc % 4) * 8;
      bK[i] = k;
      bOff[i] = (n0 + n < p.N) ? uint32_t((int64_t(k) * p.ldb + n0 + n) * 2) : kOob;
    }
  }

  auto issue = [&](int kt, int stage) {
    unsigned char *sA = smem + stage * STAGE_BYTES;
    unsigned char *sB = sA + A_BYTES;
    const int k0 = kt * BK;
    const bool live = kt < ktEnd;
#pragma unroll
    for (int i = 0; i < A_PER_W; i++) {
      const uint32_t off = (live && k0 + aCol[i] < p.K && aOff[i] != kOob)
                               ? aOff[i] + uint32_t(k0) * 2u
                               : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrcA, HOM_LDS_PTR(sA + (wave * A_PER_W + i) * 1024), 16, off, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < B_PER_W; i++) {
      uint32_t off;
      if (B_NK)
        off = (live && k0 + bK[i] < p.K && bOff[i] != kOob)
                  ? bOff[i] + uint32_t(k0) * 2u
                  : kOob;
      else
        off = (live && k0 + bK[i] < p.K && bOff[i] != kOob)
                  ? bOff[i] + uint32_t(int64_t(k0) * p.ldb * 2)
                  : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrcB, HOM_LDS_PTR(sB + (wave * B_PER_W + i) * 1024), 16, off, 0, 0, 0);
    }
  };

  float16v acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[i][j][e] = 0.f;

  // ---- fragment addresses (bytes inside a stage), constant over the walk ----
  // A: row r = waveM*WTM + i*32 + l32, logical chunk kk*2 + kb.
  const int aRow0 = waveM * WTM + l32;
  // B (row-major): transposing read.  Source lane L = lane%16 of a 16-lane
  // group supplies row kbase + L/4, 4 columns at (L%4)*4; the group's 16 columns
  // start at ((lane%32)/16)*16 of the 32-wide block.
  const int trRow = (lane % 16) / 4;
  const int trCol = ((lane % 32) / 16) * 16 + (lane % 4) * 4;

  // Fragments of one 16-wide k step of a stage, into registers.
  auto loadFrags = [&](int stage, int kk, half8 (&fa)[MI], half8 (&fb)[NI]) {
    const unsigned char *sA = smem + stage * STAGE_BYTES;
    const unsigned char *sB = sA + A_BYTES;
#pragma unroll
    for (int i = 0; i < MI; i++) {
      const int r = aRow0 + i * 32;
      fa[i] = *reinterpret_cast<const half8 *>(sA + r * 128 +
                                               swzK(r, kk * 2 + kb) * 16);
    }
    if (B_NK) {
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int r = waveN * WTN + j * 32 + l32;
        fb[j] = *reinterpret_cast<const half8 *>(sB + r * 128 +
                                                 swzK(r, kk * 2 + kb) * 16);
      }
    } else {
#pragma unroll
      for (int j = 0; j < NI; j++) {
        const int n = waveN * WTN + j * 32 + trCol;
        short4v t[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int k = kk * 16 + kb * 8 + h * 4 + trRow;
          const unsigned char *src =
              sB + k * B_ROW_BYTES + swzN<BN>(k, n / 32) * 64 + (n % 32) * 2;
          t[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) short4v *)(src));
        }
        typedef short short8v __attribute__((ext_vector_type(8)));
        short8v both;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          both[e] = t[0][e];
          both[4 + e] = t[1][e];
        }
        fb[j] = __builtin_bit_cast(half8, both);
      }
    }
  };
  auto mfmaStep = [&](half8 (&fa)[MI], half8 (&fb)[NI]) {
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int j = 0; j < NI; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i],
                                                           acc[i][j], 0, 0, 0);
  };

  // ---- main loop: NS-deep ring of slabs, one barrier per slab ----
  // Every wavefront issues exactly LOADS_PER_TILE DMA loads per slab (slabs past
  // the end are all out of range and write zeros), so "slab i+1 has landed" is
  // vmcnt <= (NS-2) * LOADS_PER_TILE once slabs up to i+NS-1 have been issued.
  // Inside a slab the fragments of k step kk+1 are fetched from LDS before the
  // MFMAs of step kk are issued (two register sets), and the barrier that frees
  // the slab's LDS buffer sits between the last fragment fetch and the last
  // MFMA group, so the matrix core keeps running while the wavefronts
  // synchronise, refill the ring and fetch the next slab's first fragments.
  // The waits and the barrier are one opaque asm statement with a memory
  // clobber: the compiler may not move LDS reads or DMA issues across it.
  constexpr int kInFlight = (NS - 2) * LOADS_PER_TILE;
  constexpr int KSTEPS = BK / 16;
  half8 fa[2][MI], fb[2][NI];
#pragma unroll
  for (int s = 0; s < NS - 1; s++)
    issue(ktBegin + s, s);
  const int nk = ktEnd - ktBegin;
  if (nk > 0) {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kInFlight) : "memory");
    issue(ktBegin + NS - 1, NS - 1);
    loadFrags(0, 0, fa[0], fb[0]);
    for (int i = 0; i < nk; i++) {
      const int cur = i % NS;
#pragma unroll
      for (int kk = 0; kk < KSTEPS - 1; kk++) {
        loadFrags(cur, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
        mfmaStep(fa[kk & 1], fb[kk & 1]);
      }
      if (i + 1 < nk) {
        // all of this wavefront's reads of slab i are in registers; slab i+1
        // has landed for this wavefront; then wait for the other wavefronts
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(
                         kInFlight)
                     : "memory");
        issue(ktBegin + i + NS, cur);
        loadFrags((i + 1) % NS, 0, fa[0], fb[0]);
      }
      mfmaStep(fa[(KSTEPS - 1) & 1], fb[(KSTEPS - 1) & 1]);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // no DMA may outlive the loop

  if (numSlices > 1) {
    storePartial<MI, NI, THREADS>(p, acc, tile, slice, numSlices, tid);
    return;
  }
  static_assert(WM * WN * 32 * (WTN * 4 + 16) <= 2 * STAGE_BYTES,
                "epilogue strips must fit the main loop's LDS");
  epilogueStoreLds<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane,
                                          wave, smem);
#endif
}

// ==================================================================== pipe ==
// Same LDS layout, fragment reads and barrier placement as the dma kernels, but
// the slabs travel global -> registers -> LDS (two LDS buffers): the loads of
// slab i+1 are issued before slab i is multiplied and written to LDS after it.
// The vector memory path into registers sustains several times the bandwidth
// of the LDS-DMA path on this chip, which matters once a CU streams more than
// ~16 bytes per clock (large tiles, or several workgroups per CU).
template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK>
__global__ __launch_bounds__(WM *WN *kWave) void gemmPipeKernel(GemmParams p) {
  static_assert(DIST >= 1, "at least one slab of global loads in flight");
  constexpr int BK = 64;
  constexpr int THREADS = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 32, NI = WTN / 32;
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_VECS = A_BYTES / 16, B_VECS = B_BYTES / 16;
  static_assert(A_VECS % THREADS == 0 && B_VECS % THREADS == 0,
                "tile must split evenly over the threads");
  constexpr int A_PER_T = A_VECS / THREADS, B_PER_T = B_VECS / THREADS;
  constexpr int B_ROW_BYTES = B_NK ? 128 : BN * 2;
  constexpr int B_VPR = B_ROW_BYTES / 16; // vectors per LDS row of B
  constexpr int KSTEPS = BK / 16;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int waveM = wave / WN, waveN = wave % WN;
  const int l32 = lane % 32, kb = lane / 32;

  // Persistent over tiles: the grid holds at most as many workgroups as fit on
  // the chip at once and each walks tiles pid, pid + grid, ...  (the grid is a
  // multiple of the XCD count, so a workgroup's tiles stay in its XCD's
  // contiguous range).  A tile's output stores drain and the next tile's first
  // slabs arrive while other work runs, instead of between two workgroups.
  const int nTiles = p.tilesM * p.tilesN;
  for (int vpid = blockIdx.x; vpid < nTiles; vpid += gridDim.x) {
  if (vpid != int(blockIdx.x))
    __syncthreads(); // the previous tile's epilogue strips live in this LDS
  const int tile = tileForBlock(nTiles, vpid);
  int tileM, tileN;
  tileCoords(tile, p.tilesM, p.tilesN, &tileM, &tileN);
  const int m0 = tileM * BM, n0 = tileN * BN;
  const int slice = blockIdx.y, numSlices = gridDim.y;
  const int kTiles = (p.K + BK - 1) / BK;
  const int ktBegin = slice * p.kTilesPerSlice;
  int ktEnd = ktBegin + p.kTilesPerSlice;
  if (ktEnd > kTiles)
    ktEnd = kTiles;

  // ---- global sources ----
  // Buffer loads from descriptors based at this tile's first row (A) / first
  // row or column block (B): a constant 32-bit byte offset per thread plus a
  // scalar offset per slab.  Rows / columns past the edge are clamped to the
  // last valid one: what they fetch only reaches outputs that are never
  // stored.  Every slab issues the same number of loads and there is no branch
  // around a load, so the compiler's outstanding-load counts are exact (a
  // branch makes it wait for everything in flight and defeats the pipeline).
  // The main loop walks the slice's FULL slabs only and asks for no range
  // test per vector: vector instructions in that loop cost matrix-core time.
  // A slab requested past the last full one is replaced by the last full one
  // (it is never used), and a partial last slab (K not a multiple of 64) is
  // multiplied ahead of the loop by a short unpipelined pass whose loads map
  // vectors at or past kEnd to an offset outside the descriptor (they read as
  // zero without touching memory).
  constexpr uint32_t kOob = 0x80000000u;
  auto clampBytes = [](int64_t b) -> int32_t {
    return b > 0x7fffffffLL ? 0x7fffffff : (b < 0 ? 0 : int32_t(b));
  };
  const _Float16 *aTile = p.A + int64_t(m0) * p.lda;
  const auto rsrcA = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(aTile), 0,
      clampBytes(int64_t(p.M - m0) * p.lda * 2), 0x00020000);
  const _Float16 *bTile = B_NK ? p.B + int64_t(n0) * p.ldb : p.B + n0;
  const auto rsrcB = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(bTile), 0,
      clampBytes(B_NK ? int64_t(p.N - n0) * p.ldb * 2
                      : (int64_t(p.K) * p.ldb - n0) * 2),
      0x00020000);
  const int kEnd = ktEnd * BK < p.K ? ktEnd * BK : p.K;
  uint32_t aOff[A_PER_T], bOff[B_PER_T];
  // LDS destination of vector i = destination of vector 0 + i * DST_STEP: the
  // row advances by a multiple of 16 per vector, which leaves both swizzles
  // unchanged (they depend on row bits 0..3 only).
  constexpr int DST_STEP = THREADS * 16;
  static_assert((THREADS / 8) % 16 == 0 && (THREADS / B_VPR) % 4 == 0 &&
                    (BN != 64 || (THREADS / B_VPR) % 4 == 0),
                "vector step must preserve the LDS swizzles");
  int aDst0 = 0, bDst0 = 0;
  int aK[A_PER_T], bK[B_PER_T]; // k position inside the slab
#pragma unroll
  for (int i = 0; i < A_PER_T; i++) {
    const int v = tid + i * THREADS;
    const int r = v / 8, c = v % 8;
    const int rr = m0 + r < p.M ? r : p.M - 1 - m0;
    aK[i] = c * 8;
    aOff[i] = (uint32_t(rr) * uint32_t(p.lda) + c * 8) * 2u;
    if (i == 0)
      aDst0 = r * 128 + swzK(r, c) * 16;
  }
#pragma unroll
  for (int i = 0; i < B_PER_T; i++) {
    const int v = tid + i * THREADS;
    const int r = v / B_VPR, c = v % B_VPR;
    if (B_NK) {
      const int rr = n0 + r < p.N ? r : p.N - 1 - n0;
      bK[i] = c * 8;
      bOff[i] = (uint32_t(rr) * uint32_t(p.ldb) + c * 8) * 2u;
      if (i == 0)
        bDst0 = r * 128 + swzK(r, c) * 16;
    } else {
      const int cc = n0 + c * 8 < p.N ? c * 8 : p.N - 8 - n0;
      bK[i] = r;
      bOff[i] = (uint32_t(r) * uint32_t(p.ldb) + cc) * 2u;
      if (i == 0)
        bDst0 = r * B_ROW_BYTES + swzN<BN>(r, c / 4) * 64 + (c % 4) * 16;
    }
  }

  half8 regA[DIST][A_PER_T], regB[DIST][B_PER_T];
  // Slabs of this slice that lie inside [0, kEnd) entirely, and whether a
  // partial one follows them (only the last slice of a ragged K has one).
  const int nkFull = (kEnd - ktBegin * BK) / BK;
  const bool hasTail = kEnd - ktBegin * BK > nkFull * BK;
  const int ktLastFull = ktBegin + nkFull - 1;
  // Full slab kt (requests past the last full slab fetch that one again).
  auto loadGlobal = [&](int kt, auto setC) {
    constexpr int S = decltype(setC)::value;
    const int k0 = (kt < ktLastFull ? kt : ktLastFull) * BK;
    const uint32_t sA = uint32_t(k0) * 2u;
    const uint32_t sB = B_NK ? sA : uint32_t(k0) * uint32_t(p.ldb) * 2u;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++)
      regA[S][i] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, aOff[i], sA, 0));
#pragma unroll
    for (int i = 0; i < B_PER_T; i++)
      regB[S][i] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcB, bOff[i], sB, 0));
  };
  // Slab kt with a range test per vector (the partial slab).
  auto loadGlobalChecked = [&](int kt, auto setC) {
    constexpr int S = decltype(setC)::value;
    const int k0 = kt * BK;
    const uint32_t sA = uint32_t(k0) * 2u;
    const uint32_t sB = B_NK ? sA : uint32_t(k0) * uint32_t(p.ldb) * 2u;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++)
      regA[S][i] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(
                     rsrcA, k0 + aK[i] < kEnd ? aOff[i] : kOob, sA, 0));
#pragma unroll
    for (int i = 0; i < B_PER_T; i++)
      regB[S][i] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(
                     rsrcB, k0 + bK[i] < kEnd ? bOff[i] : kOob, sB, 0));
  };
  auto storeLds = [&](int stage, auto setC) {
    constexpr int S = decltype(setC)::value;
    unsigned char *sA = smem + stage * STAGE_BYTES;
    unsigned char *sB = sA + A_BYTES;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++)
      *reinterpret_cast<half8 *>(sA + aDst0 + i * DST_STEP) = regA[S][i];
#pragma unroll
    for (int i = 0; i < B_PER_T; i++)
      *reinterpret_cast<half8 *>(sB + bDst0 + i * DST_STEP) = regB[S][i];
  };

  float16v acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[i][j][e] = 0.f;

  // ---- fragment addresses: a few per-lane bases, the rest are immediates ----
  // K-contiguous tiles: the swizzle term (row >> 1) & 7 only involves bits of
  // lane % 32 (wave / block offsets are multiples of 32), so the chunk position
  // of k step kk is the same for every 32-row block of the wavefront.
  const int swzLane = (l32 >> 1) & 7;
  int aFrag[KSTEPS], bFragK[KSTEPS];
#pragma unroll
  for (int kk = 0; kk < KSTEPS; kk++) {
    aFrag[kk] = (waveM * WTM + l32) * 128 + ((kk * 2 + kb) ^ swzLane) * 16;
    bFragK[kk] =
        A_BYTES + (waveN * WTN + l32) * 128 + ((kk * 2 + kb) ^ swzLane) * 16;
  }
  // Row-major B, transposing reads: source lane L = lane % 16 of a 16-lane group
  // supplies row kbase + L/4 and the 4 columns at (L%4)*4 of the group's 16
  // columns.  k & 3 == L/4 for every (kk, kb, h), so the 64-byte group swizzle
  // is a per-lane constant as well.
  const int trRow = (lane % 16) / 4;
  const int trCol = ((lane % 32) / 16) * 16 + (lane % 4) * 4;
  int bFragN[NI];
#pragma unroll
  for (int j = 0; j < NI; j++) {
    const int group = (waveN * WTN) / 32 + j;
    bFragN[j] = A_BYTES + (kb * 8 + trRow) * B_ROW_BYTES +
                swzN<BN>(trRow, group) * 64 + trCol * 2;
  }

  // One fragment per call: unit u < MI is A block u, the rest are B blocks.
  auto loadFragUnit = [&](int stage, int kk, half8 (&fa)[MI], half8 (&fb)[NI],
                          auto uC) {
    constexpr int U = decltype(uC)::value;
    const unsigned char *st = smem + stage * STAGE_BYTES;
    if constexpr (U < MI) {
      fa[U] = *reinterpret_cast<const half8 *>(st + aFrag[kk] + U * 32 * 128);
    } else if constexpr (B_NK) {
      constexpr int j = U - MI;
      fb[j] = *reinterpret_cast<const half8 *>(st + bFragK[kk] + j * 32 * 128);
    } else {
      constexpr int j = U - MI;
      short4v t[2];
#pragma unroll
      for (int h = 0; h < 2; h++)
        t[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) short4v *)(
                st + bFragN[j] + (kk * 16 + h * 4) * B_ROW_BYTES));
      typedef short short8v __attribute__((ext_vector_type(8)));
      short8v both;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        both[e] = t[0][e];
        both[4 + e] = t[1][e];
      }
      fb[j] = __builtin_bit_cast(half8, both);
    }
  };
  auto loadFrags = [&](int stage, int kk, half8 (&fa)[MI], half8 (&fb)[NI]) {
    staticFor<MI + NI>([&](auto uC) { loadFragUnit(stage, kk, fa, fb, uC); });
  };

  // ---- main loop ----
  // LDS holds slab i (buffer i & 1); slabs i+1 .. i+DIST sit in registers or are
  // on their way there, slab s in register set s % DIST.  While slab i is
  // multiplied, slab i+1 moves from its register set to the other LDS buffer
  // one 16-byte vector at a time, and each vector's registers are refilled
  // with slab i+1+DIST right behind the LDS write.  These LDS writes and global
  // loads are spread between the MFMAs of the first KSTEPS-1 k steps
  // (scheduling barriers pin the order): issued as one burst they fill the
  // memory pipelines' queues, the wavefront blocks on issue, and with both
  // wavefronts of a SIMD in the same phase the matrix core idles for as long as
  // the burst takes to drain.  The loop is unrolled DIST times to keep the
  // register-set index a compile-time constant.
  // The barrier is a bare s_barrier behind an LDS-only wait: a fence here would
  // drain the global loads that were just issued.
  // The fragments of k step kk+1 are fetched under the MFMAs of step kk (two
  // fragment sets).
  constexpr int NV = A_PER_T + B_PER_T; // vectors per thread and slab
  constexpr int NM = MI * NI;           // MFMAs per wavefront and k step
  constexpr int ST_STEPS = KSTEPS - 1;  // k steps that carry staging work
  half8 fa[2][MI], fb[2][NI];
  const int nk = nkFull; // the pipelined loop walks the full slabs
  // Moves vector v of register set S to LDS and refills it from full slab kt
  // (already clamped to the last full slab by the caller).
  auto stageVec = [&](int stage, int kt, auto setC, auto vC) {
    constexpr int S = decltype(setC)::value;
    constexpr int V = decltype(vC)::value;
    unsigned char *sA = smem + stage * STAGE_BYTES;
    unsigned char *sB = sA + A_BYTES;
    const int k0 = kt * BK;
    if constexpr (V < A_PER_T) {
      *reinterpret_cast<half8 *>(sA + aDst0 + V * DST_STEP) = regA[S][V];
      regA[S][V] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, aOff[V],
                                                       uint32_t(k0) * 2u, 0));
    } else {
      constexpr int W = V - A_PER_T;
      *reinterpret_cast<half8 *>(sB + bDst0 + W * DST_STEP) = regB[S][W];
      regB[S][W] = __builtin_bit_cast(
          half8,
          __builtin_amdgcn_raw_buffer_load_b128(
              rsrcB, bOff[W],
              B_NK ? uint32_t(k0) * 2u : uint32_t(k0) * uint32_t(p.ldb) * 2u,
              0));
    }
  };
  // The MFMAs of one k step on fragments (a, b).  Spread between them: the
  // fragment reads of another k step (rdStage, rdKk) into (na, nb) when RD, and
  // the staging vectors [V0, V1) when stageOn.  Memory operation q of n goes in
  // front of MFMA q * NM / n.
  auto mfmaMixed = [&](half8 (&a)[MI], half8 (&b)[NI], half8 (&na)[MI],
                       half8 (&nb)[NI], int rdStage, int rdKk, auto rdC,
                       int stStage, int kt, bool stageOn, auto setC, auto v0C,
                       auto v1C) {
    constexpr bool RD = decltype(rdC)::value;
    constexpr int V0 = decltype(v0C)::value, V1 = decltype(v1C)::value;
    constexpr int NR = RD ? MI + NI : 0;
    constexpr int N = NR + (V1 - V0);
    staticFor<NM>([&](auto mC) {
      constexpr int m = decltype(mC)::value;
      if constexpr (N > 0) {
        staticFor<N>([&](auto qC) {
          constexpr int q = decltype(qC)::value;
          if constexpr (q * NM / N == m) {
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (q < NR) {
              loadFragUnit(rdStage, rdKk, na, nb,
                           std::integral_constant<int, (q < NR ? q : 0)>{});
            } else {
              if (stageOn)
                stageVec(stStage, kt, setC,
                         std::integral_constant<int, V0 + q - NR>{});
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        });
      }
      acc[m / NI][m % NI] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
          b[m % NI], a[m / NI], acc[m / NI][m % NI], 0, 0, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  // tailC: the slab may be the last one (then nothing follows it); the
  // steady-state loop knows it is not and runs without branches.
  auto slab = [&](int i, auto setC, auto tailC) {
    constexpr bool kTail = decltype(tailC)::value;
    const int cur = i & 1;
    const bool more = !kTail || i + 1 < nk;
    const int ktWant = ktBegin + i + 1 + DIST;
    const int ktNext = ktWant < ktLastFull ? ktWant : ktLastFull;
    staticFor<KSTEPS>([&](auto kkC) {
      constexpr int kk = decltype(kkC)::value;
      constexpr int V0 = kk < ST_STEPS ? kk * NV / ST_STEPS : NV;
      constexpr int V1 = kk < ST_STEPS ? (kk + 1) * NV / ST_STEPS : NV;
      using V0C = std::integral_constant<int, V0>;
      using V1C = std::integral_constant<int, V1>;
      constexpr int cs = kk % 2, ns = (kk + 1) % 2;
      if constexpr (kk < KSTEPS - 1) {
        mfmaMixed(fa[cs], fb[cs], fa[ns], fb[ns], cur, kk + 1, std::true_type{},
                  cur ^ 1, ktNext, more, setC, V0C{}, V1C{});
      } else {
        static_assert(ns == 0, "the next slab finds its first fragments in set 0");
        if (more) {
          // Every wavefront has its last fragments of slab i in registers and
          // slab i+1 is complete in the other buffer after this barrier; its
          // first fragments arrive under the MFMAs of the last k step.
          asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
          mfmaMixed(fa[cs], fb[cs], fa[ns], fb[ns], cur ^ 1, 0, std::true_type{},
                    0, 0, false, setC, V0C{}, V1C{});
        } else {
          mfmaMixed(fa[cs], fb[cs], fa[ns], fb[ns], 0, 0, std::false_type{}, 0,
                    0, false, setC, V0C{}, V1C{});
        }
      }
    });
  };
  if (hasTail) {
    // The partial slab, unpipelined: it is one slab of a ragged problem.
    using Set0 = std::integral_constant<int, 0>;
    loadGlobalChecked(ktBegin + nkFull, Set0{});
    storeLds(0, Set0{});
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KSTEPS; kk++) {
      loadFrags(0, kk, fa[0], fb[0]);
#pragma unroll
      for (int m = 0; m < NM; m++)
        acc[m / NI][m % NI] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            fb[0][m % NI], fa[0][m / NI], acc[m / NI][m % NI], 0, 0, 0);
    }
    __syncthreads(); // buffer 0 is rewritten by the first full slab
  }
  if (nk > 0) {
    staticFor<DIST>(
        [&](auto d) { loadGlobal(ktBegin + decltype(d)::value, d); });
    storeLds(0, std::integral_constant<int, 0>{});
    loadGlobal(ktBegin + DIST, std::integral_constant<int, 0>{});
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    loadFrags(0, 0, fa[0], fb[0]);
    int i = 0;
    for (; i + DIST < nk; i += DIST) {
      staticFor<DIST>([&](auto d) {
        constexpr int D = decltype(d)::value;
        slab(i + D, std::integral_constant<int, (D + 1) % DIST>{},
             std::false_type{});
      });
    }
    bool go = true;
    staticFor<DIST>([&](auto d) {
      constexpr int D = decltype(d)::value;
      go = go && i + D < nk;
      if (go)
        slab(i + D, std::integral_constant<int, (D + 1) % DIST>{},
             std::true_type{});
    });
  }

  if (numSlices > 1) {
    storePartial<MI, NI, THREADS>(p, acc, tile, slice, numSlices, tid);
    continue;
  }
  static_assert(WM * WN * 32 * (WTN * 4 + 16) <= 2 * STAGE_BYTES,
                "epilogue strips must fit the main loop's LDS");
  epilogueStoreLds<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane,
                                          wave, smem);
  } // tiles of this workgroup
}

// ================================================================== staged ==
// VEC == 8: N, K multiples of 8 and 16-byte aligned operands (128-bit global
// accesses).  VEC == 1: any shape/alignment, scalar global accesses.
template <int BM, int BN, int BK, int WM, int WN, int EPI, bool B_NK, int VEC>
__global__ __launch_bounds__(WM *WN *kWave) void gemmStagedKernel(GemmParams p) {
  constexpr int kThreads = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 32, NI = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be 32-aligned");
  static_assert(BK % 16 == 0, "BK must be a multiple of the MFMA k (16)");
  constexpr int A_LD = BK + 8;  // halves per LDS row of A (and of B when NK)
  constexpr int BP_LD = BN + 8; // dwords per LDS row of k-pair-packed B
  constexpr int A_BYTES = BM * A_LD * 2;
  constexpr int B_BYTES = B_NK ? BN * A_LD * 2 : (BK / 2) * BP_LD * 4;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int waveM = wave / WN, waveN = wave % WN;

  const int nTiles = p.tilesM * p.tilesN;
  const int tile = tileForBlock(nTiles, blockIdx.x);
  int tileM, tileN;
  tileCoords(tile, p.tilesM, p.tilesN, &tileM, &tileN);
  const int m0 = tileM * BM, n0 = tileN * BN;
  const int slice = blockIdx.y, numSlices = gridDim.y;

  const int kTiles = (p.K + BK - 1) / BK;
  const int ktBegin = slice * p.kTilesPerSlice;
  int ktEnd = ktBegin + p.kTilesPerSlice;
  if (ktEnd > kTiles)
    ktEnd = kTiles;

  float16v acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        acc[i][j][e] = 0.f;

  constexpr int A_VECS = BM * BK / 8;
  constexpr int A_PER_T = (A_VECS + kThreads - 1) / kThreads;
  constexpr int A_VPR = BK / 8;
  constexpr int BNK_VECS = BN * BK / 8;
  constexpr int BNK_PER_T = (BNK_VECS + kThreads - 1) / kThreads;
  constexpr int BKN_ITEMS = (BK / 2) * (BN / 8); // (k-pair, 8 columns)
  constexpr int BKN_PER_T = (BKN_ITEMS + kThreads - 1) / kThreads;
  constexpr int BKN_CPR = BN / 8;

  half8 regA[VEC == 8 ? A_PER_T : 1];
  half8 regB0[VEC == 8 ? (B_NK ? BNK_PER_T : BKN_PER_T) : 1];
  half8 regB1[VEC == 8 ? (B_NK ? 1 : BKN_PER_T) : 1];

  auto zero8 = []() {
    half8 z;
#pragma unroll
    for (int e = 0; e < 8; e++)
      z[e] = _Float16(0);
    return z;
  };

  auto loadGlobal = [&](int kt) {
    if (VEC != 8)
      return;
    const int k0 = kt * BK;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++) {
      const int v = tid + i * kThreads;
      const int r = v / A_VPR, c = (v % A_VPR) * 8;
      half8 val = zero8();
      if (v < A_VECS && m0 + r < p.M && k0 + c < p.K)
        val = *reinterpret_cast<const half8 *>(p.A + int64_t(m0 + r) * p.lda +
                                               k0 + c);
      regA[i] = val;
    }
    if (B_NK) {
#pragma unroll
      for (int i = 0; i < BNK_PER_T; i++) {
        const int v = tid + i * kThreads;
        const int r = v / A_VPR, c = (v % A_VPR) * 8;
        half8 val = zero8();
        if (v < BNK_VECS && n0 + r < p.N && k0 + c < p.K)
          val = *reinterpret_cast<const half8 *>(
              p.B + int64_t(n0 + r) * p.ldb + k0 + c);
        regB0[i] = val;
      }
    } else {
#pragma unroll
      for (int i = 0; i < BKN_PER_T; i++) {
        const int v = tid + i * kThreads;
        const int kp = v / BKN_CPR, c = (v % BKN_CPR) * 8;
        half8 v0 = zero8(), v1 = zero8();
        if (v < BKN_ITEMS && n0 + c < p.N) {
          const int k = k0 + 2 * kp;
          if (k < p.K)
            v0 = *reinterpret_cast<const half8 *>(p.B + int64_t(k) * p.ldb +
                                                  n0 + c);
          if (k + 1 < p.K)
            v1 = *reinterpret_cast<const half8 *>(p.B + int64_t(k + 1) * p.ldb +
                                                  n0 + c);
        }
        regB0[i] = v0;
        regB1[i] = v1;
      }
    }
  };

  auto storeLds = [&](int stage) {
    unsigned char *base = smem + stage * STAGE_BYTES;
    _Float16 *sA = reinterpret_cast<_Float16 *>(base);
    if (VEC != 8)
      return;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++) {
      const int v = tid + i * kThreads;
      const int r = v / A_VPR, c = (v % A_VPR) * 8;
      if (v < A_VECS)
        *reinterpret_cast<half8 *>(sA + r * A_LD + c) = regA[i];
    }
    if (B_NK) {
      _Float16 *sB = reinterpret_cast<_Float16 *>(base + A_BYTES);
#pragma unroll
      for (int i = 0; i < BNK_PER_T; i++) {
        const int v = tid + i * kThreads;
        const int r = v / A_VPR, c = (v % A_VPR) * 8;
        if (v < BNK_VECS)
          *reinterpret_cast<half8 *>(sB + r * A_LD + c) = regB0[i];
      }
    } else {
      uint32_t *sB = reinterpret_cast<uint32_t *>(base + A_BYTES);
#pragma unroll
      for (int i = 0; i < BKN_PER_T; i++) {
        const int v = tid + i * kThreads;
        const int kp = v / BKN_CPR, c = (v % BKN_CPR) * 8;
        if (v < BKN_ITEMS) {
          half8 lo, hi; // (k, k+1) pairs for columns c..c+3 and c+4..c+7
#pragma unroll
          for (int e = 0; e < 4; e++) {
            lo[2 * e] = regB0[i][e];
            lo[2 * e + 1] = regB1[i][e];
            hi[2 * e] = regB0[i][4 + e];
            hi[2 * e + 1] = regB1[i][4 + e];
          }
          *reinterpret_cast<half8 *>(sB + kp * BP_LD + c) = lo;
          *reinterpret_cast<half8 *>(sB + kp * BP_LD + c + 4) = hi;
        }
      }
    }
  };

  // Scalar staging straight into LDS for unaligned problems.
  auto stageScalar = [&](int kt, int stage) {
    unsigned char *base = smem + stage * STAGE_BYTES;
    _Float16 *sA = reinterpret_cast<_Float16 *>(base);
    const int k0 = kt * BK;
    for (int idx = tid; idx < BM * BK; idx += kThreads) {
      const int r = idx / BK, c = idx % BK;
      _Float16 val = _Float16(0);
      if (m0 + r < p.M && k0 + c < p.K)
        val = p.A[int64_t(m0 + r) * p.lda + k0 + c];
      sA[r * A_LD + c] = val;
    }
    if (B_NK) {
      _Float16 *sB = reinterpret_cast<_Float16 *>(base + A_BYTES);
      for (int idx = tid; idx < BN * BK; idx += kThreads) {
        const int r = idx / BK, c = idx % BK;
        _Float16 val = _Float16(0);
        if (n0 + r < p.N && k0 + c < p.K)
          val = p.B[int64_t(n0 + r) * p.ldb + k0 + c];
        sB[r * A_LD + c] = val;
      }
    } else {
      _Float16 *sB = reinterpret_cast<_Float16 *>(base + A_BYTES);
      for (int idx = tid; idx < BK * BN; idx += kThreads) {
        const int k = idx / BN, n = idx % BN;
        _Float16 val = _Float16(0);
        if (k0 + k < p.K && n0 + n < p.N)
          val = p.B[int64_t(k0 + k) * p.ldb + n0 + n];
        sB[((k >> 1) * BP_LD + n) * 2 + (k & 1)] = val;
      }
    }
  };

  auto compute = [&](int stage) {
    const unsigned char *base = smem + stage * STAGE_BYTES;
    const _Float16 *sA = reinterpret_cast<const _Float16 *>(base);
    const int l32 = lane % 32, kb = lane / 32;
#pragma unroll
    for (int kk = 0; kk < BK / 16; kk++) {
      half8 fa[MI], fb[NI];
#pragma unroll
      for (int i = 0; i < MI; i++) {
        const int r = waveM * WTM + i * 32 + l32;
        fa[i] = *reinterpret_cast<const half8 *>(sA + r * A_LD + kk * 16 +
                                                 kb * 8);
      }
      if (B_NK) {
        const _Float16 *sB = reinterpret_cast<const _Float16 *>(base + A_BYTES);
#pragma unroll
        for (int j = 0; j < NI; j++) {
          const int c = waveN * WTN + j * 32 + l32;
          fb[j] = *reinterpret_cast<const half8 *>(sB + c * A_LD + kk * 16 +
                                                   kb * 8);
        }
      } else {
        const uint32_t *sB = reinterpret_cast<const uint32_t *>(base + A_BYTES);
#pragma unroll
        for (int j = 0; j < NI; j++) {
          const int c = waveN * WTN + j * 32 + l32;
          const int kp = kk * 8 + kb * 4;
          uint4v w;
#pragma unroll
          for (int e = 0; e < 4; e++)
            w[e] = sB[(kp + e) * BP_LD + c];
          fb[j] = __builtin_bit_cast(half8, w);
        }
      }
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i],
                                                             acc[i][j], 0, 0, 0);
    }
  };

  if (ktBegin < ktEnd) {
    if (VEC == 8) {
      loadGlobal(ktBegin);
      storeLds(0);
    } else {
      stageScalar(ktBegin, 0);
    }
    __syncthreads();
    for (int kt = ktBegin; kt < ktEnd; kt++) {
      const int cur = (kt - ktBegin) & 1;
      const bool more = kt + 1 < ktEnd;
      if (VEC == 8) {
        if (more)
          loadGlobal(kt + 1);
        compute(cur);
        if (more)
          storeLds(cur ^ 1);
      } else {
        if (more)
          stageScalar(kt + 1, cur ^ 1);
        compute(cur);
      }
      __syncthreads();
    }
  }

  if (numSlices > 1) {
    storePartial<MI, NI, kThreads>(p, acc, tile, slice, numSlices, tid);
    return;
  }
  epilogueStore<MI, NI, WTM, WTN, EPI, VEC>(p, acc, m0, n0, waveM, waveN, lane);
}

// ------------------------------------------------------- layer-norm pair --
// Row-statistic partials [pieces][M] (sum, sum of squares) -> var / mean in the
// form the pair exchanges (Layernorm.h:166-192 of the reference: the second
// moment minus the squared mean, no shift).  Four lanes per row, 16 apart in
// the wavefront so that 16 neighbouring lanes read 16 neighbouring rows; each
// takes every fourth piece, four loads in flight.
__global__ __launch_bounds__(256) void rowStatsFinalizeKernel(
    const float *__restrict__ partials, int pieces, int M, int N, float eps,
    _Float16 *__restrict__ var, _Float16 *__restrict__ mean) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int q = lane / 16;
  const int m = (blockIdx.x * 4 + wave) * 16 + lane % 16;
  const int mc = m < M ? m : M - 1;
  float s = 0.f, sq = 0.f;
  for (int pc = q; pc < pieces; pc += 16) {
    float2v v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int pu = pc + 4 * u;
      v[u] = pu < pieces ? *reinterpret_cast<const float2v *>(
                               partials + (int64_t(pu) * M + mc) * 2)
                         : float2v{0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      s += v[u][0];
      sq += v[u][1];
    }
  }
  s = pairSum(rowPairSum(s));
  sq = pairSum(rowPairSum(sq));
  if (q == 0 && m < M) {
    const float mu = s / float(N);
    const float rstd = 1.0f / sqrtf(sq / float(N) - mu * mu + eps);
    var[m] = _Float16(rstd);
    mean[m] = _Float16(-mu * rstd);
  }
}

// Partial column sums of row-major B [K, N]: workgroup (x, y) sums rows
// [y * kPer, (y + 1) * kPer) of columns [32 x, 32 x + 32) into out[y][n].  A
// thread reads 8 columns of every 64th row; the 64 row phases meet in LDS.
__global__ __launch_bounds__(256) void colSumKernel(
    const _Float16 *__restrict__ B, int64_t ldb, int K, int N, int kPer,
    float *__restrict__ out) {
  __shared__ float part[64][33];
  const int tid = threadIdx.x;
  const int cg = tid % 4, ph = tid / 4;
  const int n = blockIdx.x * 32 + cg * 8;
  const int kBegin = blockIdx.y * kPer;
  const int kEnd = kBegin + kPer < K ? kBegin + kPer : K;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (n < N) {
#pragma unroll 4
    for (int k = kBegin + ph; k < kEnd; k += 64) {
      const half8 v = *reinterpret_cast<const half8 *>(B + int64_t(k) * ldb + n);
#pragma unroll
      for (int e = 0; e < 8; e++)
        acc[e] += float(v[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    part[ph][cg * 8 + e] = acc[e];
  __syncthreads();
  // 64 phases -> 8 -> 1, every thread busy in the first step
  {
    const int c = tid % 32, grp = tid / 32;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; r++)
      sum += part[grp * 8 + r][c];
    __syncthreads();
    part[grp][c] = sum;
  }
  __syncthreads();
  if (tid < 32 && blockIdx.x * 32 + tid < N) {
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 8; r++)
      sum += part[r][tid];
    out[int64_t(blockIdx.y) * N + blockIdx.x * 32 + tid] = sum;
  }
}

// ------------------------------------------------------------ kernel table --
struct LaunchPlan {
  GemmParams p;
  int splitK;
  int64_t nTiles;
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
  p.workspace = nullptr;
  if (splitK > 1) {
    const size_t wsBytes =
        size_t(plan->nTiles) * splitK * size_t(BM) * BN * sizeof(float);
    p.workspace = static_cast<float *>(scratch(kWorkspace, wsBytes, false));
    if (!p.workspace)
      return Status::kInternal;
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
  splitKReduceKernel<BM, BN, WM, WN, EPI, VEC>
      <<<dim3((unsigned)plan.nTiles), dim3(WM * WN * kWave), 0, s>>>(
          plan.p, plan.splitK);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

template <int BM, int BN, int BK, int WM, int WN, int EPI, bool B_NK, int VEC>
Status launchStaged(const GemmProblem &pr, hipStream_t s) {
  constexpr int A_LD = BK + 8, BP_LD = BN + 8;
  constexpr int A_BYTES = BM * A_LD * 2;
  constexpr int B_BYTES = B_NK ? BN * A_LD * 2 : (BK / 2) * BP_LD * 4;
  constexpr int SMEM = 2 * (A_BYTES + B_BYTES);
  LaunchPlan plan;
  Status st = planLaunch<BM, BN, BK>(pr, &plan);
  if (st != Status::kSuccess)
    return st;
  auto kernel = gemmStagedKernel<BM, BN, BK, WM, WN, EPI, B_NK, VEC>;
  static bool attrSet = false;
  st = allowLds(kernel, SMEM, &attrSet);
  if (st != Status::kSuccess)
    return st;
  if (plan.nTiles == 0)
    return Status::kSuccess;
  kernel<<<dim3((unsigned)plan.nTiles, (unsigned)plan.splitK),
           dim3(WM * WN * kWave), SMEM, s>>>(plan.p);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  if (plan.splitK > 1)
    return launchReduce<BM, BN, WM, WN, EPI, VEC>(plan, s);
  return Status::kSuccess;
}

template <int BM, int BN, int WM, int WN, int NS, int EPI, bool B_NK>
Status launchDma(const GemmProblem &pr, hipStream_t s) {
  constexpr int SMEM = NS * (BM + BN) * 64 * 2;
  LaunchPlan plan;
  Status st = planLaunch<BM, BN, 64>(pr, &plan);
  if (st != Status::kSuccess)
    return st;
  // 32-bit DMA offsets: a row-major B slab is addressed from the matrix base.
  HOM_CHECK_RET(B_NK || pr.K * pr.ldb * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument,
                "gemm: B larger than 2 GiB is not supported by this kernel");
  HOM_CHECK_RET(int64_t(BM) * pr.lda * 2 < (int64_t(1) << 31) &&
                    int64_t(BN) * pr.ldb * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument, "gemm: leading dimension too large");
  auto kernel = gemmDmaKernel<BM, BN, WM, WN, NS, EPI, B_NK>;
  static bool attrSet = false;
  st = allowLds(kernel, SMEM, &attrSet);
  if (st != Status::kSuccess)
    return st;
  if (plan.nTiles == 0)
    return Status::kSuccess;
  kernel<<<dim3((unsigned)plan.nTiles, (unsigned)plan.splitK),
           dim3(WM * WN * kWave), SMEM, s>>>(plan.p);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  if (plan.splitK > 1)
    return launchReduce<BM, BN, WM, WN, EPI, 8>(plan, s);
  return Status::kSuccess;
}

template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK>
Status launchPipe(const GemmProblem &pr, hipStream_t s) {
  constexpr int SMEM = 2 * (BM + BN) * 64 * 2;
  LaunchPlan plan;
  Status st = planLaunch<BM, BN, 64>(pr, &plan);
  if (st != Status::kSuccess)
    return st;
  // 32-bit buffer offsets: a row-major B slab is addressed from the matrix base.
  HOM_CHECK_RET(B_NK || pr.K * pr.ldb * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument,
                "gemm: B larger than 2 GiB is not supported by this kernel");
  HOM_CHECK_RET((int64_t(BM) * pr.lda + pr.K) * 2 < (int64_t(1) << 31) &&
                    (int64_t(BN) * pr.ldb + pr.K) * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument, "gemm: leading dimension too large");
  auto kernel = gemmPipeKernel<BM, BN, WM, WN, DIST, EPI, B_NK>;
  static bool attrSet = false;
  st = allowLds(kernel, SMEM, &attrSet);
  if (st != Status::kSuccess)
    return st;
  if (plan.nTiles == 0)
    return Status::kSuccess;
  // Workgroups that fit on the chip at once (rounded down to a multiple of the
  // XCD count, which the tile order relies on); more tiles than that are walked
  // by the same workgroups.
  static int resident = 0;
  if (resident == 0) {
    int perCu = 0;
    HOM_HIP_RET(hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &perCu, kernel, WM * WN * kWave, SMEM),
                Status::kInternal);
    const int cus = deviceInfo().computeUnits > 0 ? deviceInfo().computeUnits : 256;
    resident = perCu > 0 ? perCu * cus / kNumXcd * kNumXcd : 0;
    if (resident < kNumXcd)
      resident = 1 << 30; // unknown: one workgroup per tile
  }
  int64_t gridX = plan.nTiles;
  if (gridX * plan.splitK > resident)
    gridX = std::max<int64_t>(kNumXcd, resident / plan.splitK / kNumXcd * kNumXcd);
  if (gridX > plan.nTiles)
    gridX = plan.nTiles;
  kernel<<<dim3((unsigned)gridX, (unsigned)plan.splitK), dim3(WM * WN * kWave),
           SMEM, s>>>(plan.p);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  if (plan.splitK > 1)
    return launchReduce<BM, BN, WM, WN, EPI, 8>(plan, s);
  return Status::kSuccess;
}

using LaunchFn = Status (*)(const GemmProblem &, hipStream_t);

struct KernelEntry {
  GemmKernelInfo info;
  LaunchFn nn; // B as [K, N]
  LaunchFn nt; // B as [N, K]
};

// Names follow the reference generator's scheme (python/hom_manifest.py:56-74):
// <arch>_<opclass>_<acc><instr>gemm_<type>_<tile>_<K>x<stages>_<warps>_<layout>_
// align<n>_<epilogue>; "linear"/"gelu" in the name is what activation is derived
// from (GemmRunner.h:200-206).
#define HOM_DMA_ENTRY(BM, BN, WM, WN, NS, EPI_ENUM, EPI_STR, ACT)              \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_64x" #NS "_w" #WM  \
     "x" #WN "_nn_align8_" EPI_STR,                                            \
     BM, BN, 64, WM, WN, 8, 8, ACT, EPI_ENUM},                                 \
        launchDma<BM, BN, WM, WN, NS, int(EPI_ENUM), false>,                   \
        launchDma<BM, BN, WM, WN, NS, int(EPI_ENUM), true>                     \
  }
#define HOM_DMA_TILE(BM, BN, WM, WN, NS)                                       \
  HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kLinear, "linear", 0),           \
      HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kGeluErf, "gelu", 1),        \
      HOM_DMA_ENTRY(BM, BN, WM, WN, NS, Epilogue::kGeluTanh, "gelutanh", 1)

// "r<d>" after the LDS stage count marks the register-staged pipeline with d
// slabs of global loads in flight.
#define HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, EPI_ENUM, EPI_STR, ACT)           \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_64x2r" #DIST       \
     "_w" #WM "x" #WN "_nn_align8_" EPI_STR,                                   \
     BM, BN, 64, WM, WN, 8, 2, ACT, EPI_ENUM},                                 \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), false>,                \
        launchPipe<BM, BN, WM, WN, DIST, int(EPI_ENUM), true>                  \
  }
#define HOM_PIPE_TILE(BM, BN, WM, WN, DIST)                                    \
  HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kLinear, "linear", 0),        \
      HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluErf, "gelu", 1),     \
      HOM_PIPE_ENTRY(BM, BN, WM, WN, DIST, Epilogue::kGeluTanh, "gelutanh", 1)

#define HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, EPI_ENUM, EPI_STR, ACT, VEC)      \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_" #BK "x2_w" #WM   \
     "x" #WN "_nn_align" #VEC "_" EPI_STR,                                     \
     BM, BN, BK, WM, WN, VEC, VEC, ACT, EPI_ENUM},                             \
        launchStaged<BM, BN, BK, WM, WN, int(EPI_ENUM), false, VEC>,           \
        launchStaged<BM, BN, BK, WM, WN, int(EPI_ENUM), true, VEC>             \
  }
#define HOM_STAGED_TILE(BM, BN, BK, WM, WN, VEC)                               \
  HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kLinear, "linear", 0, VEC),   \
      HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluErf, "gelu", 1,      \
                       VEC),                                                   \
      HOM_STAGED_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluTanh, "gelutanh", 1, \
                       VEC)

// Manifest order is part of the ABI: compiled modules carry indices into it.
// Append new entries at the end.
const KernelEntry kKernels[] = {
    HOM_DMA_TILE(128, 128, 2, 2, 4),
    HOM_DMA_TILE(64, 64, 2, 2, 4),
    HOM_DMA_TILE(128, 64, 2, 2, 4),
    HOM_DMA_TILE(64, 64, 2, 2, 8),
    HOM_PIPE_TILE(64, 64, 2, 2, 2),
    HOM_PIPE_TILE(64, 64, 2, 2, 4),
    HOM_PIPE_TILE(128, 64, 2, 2, 2),
    HOM_PIPE_TILE(128, 64, 2, 2, 4),
    HOM_PIPE_TILE(64, 128, 2, 2, 2),
    HOM_PIPE_TILE(64, 128, 2, 2, 4),
    HOM_PIPE_TILE(128, 128, 2, 2, 2),
    HOM_PIPE_TILE(128, 128, 2, 2, 4),
    HOM_PIPE_TILE(128, 128, 2, 4, 2),
    HOM_PIPE_TILE(128, 128, 2, 4, 4),
    HOM_PIPE_TILE(256, 128, 4, 2, 2),
    HOM_PIPE_TILE(256, 128, 4, 2, 3),
    HOM_PIPE_TILE(128, 256, 2, 4, 2),
    HOM_PIPE_TILE(128, 256, 2, 4, 3),
    HOM_PIPE_TILE(256, 256, 2, 4, 1),
    HOM_PIPE_TILE(256, 256, 2, 2, 1),
    HOM_STAGED_TILE(128, 128, 32, 2, 2, 8),
    HOM_STAGED_TILE(64, 64, 64, 2, 2, 8),
    HOM_STAGED_TILE(64, 64, 32, 2, 2, 1),
};
constexpr int kNumKernels = sizeof(kKernels) / sizeof(kKernels[0]);

// Tiles the layer-norm pair kernels exist in (square, `edge` on a side, a
// wavefront covering `pieceWidth` columns); `likeKernel` picks the nearest.
struct FusedTile {
  int edge;
  int pieceWidth;
};
FusedTile fusedTileFor(int likeKernel) {
  const GemmKernelInfo &like = kKernels[likeKernel].info;
  const int area = like.tileM * like.tileN;
  if (area >= 256 * 256)
    return {256, 64};
  if (area >= 128 * 128)
    return {128, 32};
  return {64, 32};
}
template <int EPI>
Status launchFusedTile(int likeKernel, const GemmProblem &p, hipStream_t s) {
  switch (fusedTileFor(likeKernel).edge) {
  case 256:
    return launchPipe<256, 256, 2, 4, 1, EPI, false>(p, s);
  case 128:
    return launchPipe<128, 128, 2, 4, 2, EPI, false>(p, s);
  default:
    return launchPipe<64, 64, 2, 2, 2, EPI, false>(p, s);
  }
}

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

} // namespace

int gemmKernelCount() { return kNumKernels; }
const GemmKernelInfo &gemmKernelInfo(int idx) { return kKernels[idx].info; }

Status launchGemm(int idx, const GemmProblem &p, hipStream_t s) {
  HOM_CHECK_RET(idx >= 0 && idx < kNumKernels, Status::kInvalidArgument,
                "gemm: kernel index %d outside the manifest (size %d)", idx,
                kNumKernels);
  const KernelEntry &k = kKernels[idx];
  HOM_CHECK_RET(p.M >= 0 && p.N >= 0 && p.K >= 0 &&
                    p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31) &&
                    p.K < (int64_t(1) << 31),
                Status::kInvalidArgument, "gemm: problem size out of range");
  HOM_CHECK_RET(p.splitK >= 1, Status::kInvalidArgument,
                "gemm: split-K factor must be >= 1 (got %d)", p.splitK);
  HOM_CHECK_RET(p.beta == 0.f || p.C != nullptr, Status::kInvalidArgument,
                "gemm: beta != 0 needs a source tensor");
  if (k.info.alignment == 8) {
    // What CUTLASS's can_implement() rejects: misaligned leading dimensions.
    // K-contiguous operands (A, and B given as [N, K]) are read 16 bytes at a
    // time from 16-byte aligned rows; row-major B, C and D follow alignmentN.
    const int an = k.info.alignmentN;
    auto alignedTo = [](const void *q, int bytes) {
      return (reinterpret_cast<uintptr_t>(q) & uintptr_t(bytes - 1)) == 0;
    };
    const bool ok =
        p.K % 8 == 0 && p.lda % 8 == 0 && aligned16(p.A) && p.N % an == 0 &&
        (p.bIsNK ? (p.ldb % 8 == 0 && aligned16(p.B))
                 : (p.ldb % an == 0 && alignedTo(p.B, 2 * an))) &&
        p.ldd % an == 0 && alignedTo(p.D, 2 * an) &&
        (p.beta == 0.f || (p.ldc % an == 0 && alignedTo(p.C, 2 * an)));
    HOM_CHECK_RET(ok, Status::kInvalidArgument,
                  "gemm: kernel %s needs K a multiple of 8, N and the leading "
                  "dimensions of B, C, D multiples of %d, and operands aligned "
                  "to match (M=%lld N=%lld K=%lld)",
                  k.info.name, an, (long long)p.M, (long long)p.N,
                  (long long)p.K);
  }
  if (p.M == 0 || p.N == 0)
    return Status::kSuccess;
  return (p.bIsNK ? k.nt : k.nn)(p, s);
}

bool fusedGemmFits(const GemmProblem &p) {
  return !p.bIsNK && p.M > 0 && p.N > 0 && p.K > 0 &&
         p.M < (int64_t(1) << 31) && p.N < (int64_t(1) << 31) &&
         p.K < (int64_t(1) << 31) && p.K % 8 == 0 && p.N % 8 == 0 &&
         p.lda % 8 == 0 && p.ldb % 8 == 0 && p.ldd % 8 == 0 &&
         aligned16(p.A) && aligned16(p.B) && aligned16(p.D) &&
         (p.beta == 0.f || (p.C && p.ldc % 8 == 0 && aligned16(p.C)));
}

Status launchGemmRowStats(int likeKernel, const GemmProblem &p, _Float16 *var,
                          _Float16 *mean, float eps, hipStream_t s) {
  HOM_CHECK_RET(likeKernel >= 0 && likeKernel < kNumKernels && fusedGemmFits(p),
                Status::kInvalidArgument,
                "gemm + row statistics: problem does not fit the fused kernels");
  // every tile writes all of its wavefront columns, also those past N
  const FusedTile t = fusedTileFor(likeKernel);
  const int pieces =
      int((p.N + t.edge - 1) / t.edge) * (t.edge / t.pieceWidth);
  float *partials = static_cast<float *>(
      scratch(kTemp, size_t(pieces) * size_t(p.M) * 2 * sizeof(float), false));
  if (!partials)
    return Status::kInternal;
  GemmProblem q = p;
  q.splitK = 1;
  q.rowStatPartials = partials;
  Status st = launchFusedTile<kEpiRowStats>(likeKernel, q, s);
  if (st != Status::kSuccess)
    return st;
  rowStatsFinalizeKernel<<<dim3((unsigned)((p.M + 63) / 64)), dim3(256), 0,
                           s>>>(partials, pieces, int(p.M), int(p.N), eps, var,
                                mean);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

Status launchGemmRowAffine(int likeKernel, const GemmProblem &p,
                           const _Float16 *var, const _Float16 *mean,
                           hipStream_t s) {
  HOM_CHECK_RET(likeKernel >= 0 && likeKernel < kNumKernels && fusedGemmFits(p),
                Status::kInvalidArgument,
                "layernorm + gemm: problem does not fit the fused kernels");
  // 128 rows of B per column-sum workgroup (two 16-byte loads per lane), at
  // most 16 slices
  int slices = int((p.K + 127) / 128);
  if (slices > 16)
    slices = 16;
  const int kPer = int((p.K + slices - 1) / slices);
  float *colSum = static_cast<float *>(
      scratch(kTemp, size_t(slices) * size_t(p.N) * sizeof(float), false));
  if (!colSum)
    return Status::kInternal;
  colSumKernel<<<dim3((unsigned)((p.N + 31) / 32), (unsigned)slices), dim3(256),
                 0, s>>>(p.B, p.ldb, int(p.K), int(p.N), kPer, colSum);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  GemmProblem q = p;
  q.splitK = 1;
  q.rowScale = var;
  q.rowShift = mean;
  q.colSum = colSum;
  q.colSumSlices = slices;
  return launchFusedTile<kEpiRowAffine>(likeKernel, q, s);
}

} // namespace hom
