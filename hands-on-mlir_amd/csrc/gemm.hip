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
// Kernel structure
//  * one workgroup of WM x WN wavefronts computes a BM x BN tile of D; every
//    wavefront owns a (BM/WM) x (BN/WN) sub-tile made of 32x32 MFMA blocks
//    (v_mfma_f32_32x32x16_f16: 64 lanes x 8 halves per operand, 16 fp32
//    accumulators per lane);
//  * K is walked in BK slabs that are staged global -> registers -> LDS with
//    two LDS buffers, so the loads of slab k+1 overlap the MFMAs of slab k;
//  * A is kept K-contiguous in LDS (row padded by 16 bytes, which makes the
//    128-bit fragment reads bank-conflict free).  Row-major B has N
//    contiguous, but an MFMA operand wants 8 consecutive k per lane: while
//    staging, each thread interleaves two consecutive k rows into (k, k+1)
//    half2 pairs, and a fragment is then four conflict-free 32-bit reads;
//  * the MFMA is issued with the operands swapped (B fragment first), i.e. it
//    produces the transposed block, so each lane ends up with 4 consecutive
//    columns of one row of D and the epilogue can use 64-bit accesses;
//  * split-K: gridDim.y slices of K.  Each slice stores its fp32 partial tile
//    to a workspace and bumps a per-tile arrival counter; whichever slice
//    arrives last sums all partials in slice order (deterministic) and runs the
//    epilogue, then clears the counter for the next launch.  Nothing spins.
//  * workgroup ids are remapped so that each of the 8 XCDs (which receive
//    consecutive ids round-robin and have private L2s) works on a contiguous
//    run of tiles.
#include "kernels.h"

namespace hom {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kNumXcd = 8;

struct GemmParams {
  const _Float16 *A;
  const _Float16 *B;
  const _Float16 *C;
  _Float16 *D;
  float *workspace;    // split-K partial tiles
  uint32_t *counters;  // split-K arrival counters, one per output tile
  int M, N, K;
  int64_t lda, ldb, ldc, ldd;
  int cRowPeriod;
  float alpha, beta;
  int tilesM, tilesN;
  int kTilesPerSlice;
};

__device__ __forceinline__ float geluErf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
// 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)), u = sqrt(2/pi) (x + 0.044715 x^3)
__device__ __forceinline__ float geluTanh(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return x / (1.0f + __expf(-2.0f * u));
}

template <int EPI> __device__ __forceinline__ float activate(float v) {
  if (EPI == int(Epilogue::kGeluErf))
    return geluErf(v);
  if (EPI == int(Epilogue::kGeluTanh))
    return geluTanh(v);
  return v;
}

// VEC == 8: N, K multiples of 8 and 16-byte aligned operands (128-bit global
// accesses).  VEC == 1: any shape/alignment, scalar global accesses.
template <int BM, int BN, int BK, int WM, int WN, int EPI, bool B_NK, int VEC>
__global__ __launch_bounds__(WM *WN *kWave) void gemmKernel(GemmParams p) {
  constexpr int kThreads = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN; // wavefront tile
  constexpr int MI = WTM / 32, NI = WTN / 32; // 32x32 MFMA blocks per wave
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be 32-aligned");
  static_assert(BK % 16 == 0, "BK must be a multiple of the MFMA k (16)");
  constexpr int A_LD = BK + 8;     // halves per LDS row of A (and of B when NK)
  constexpr int BP_LD = BN + 8;    // dwords per LDS row of k-pair-packed B
  constexpr int A_BYTES = BM * A_LD * 2;
  constexpr int B_BYTES = B_NK ? BN * A_LD * 2 : (BK / 2) * BP_LD * 4;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int waveM = wave / WN, waveN = wave % WN;

  // ---- tile assignment (XCD-contiguous) ----
  const int nTiles = p.tilesM * p.tilesN;
  int tile;
  {
    const int pid = blockIdx.x;
    const int q = nTiles / kNumXcd, r = nTiles % kNumXcd;
    const int xcd = pid % kNumXcd, loc = pid / kNumXcd;
    tile = xcd * q + (xcd < r ? xcd : r) + loc;
  }
  const int tileM = tile / p.tilesN, tileN = tile % p.tilesN;
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

  // ---- global -> register staging ----
  constexpr int A_VECS = BM * BK / 8;                 // 16-byte vectors of A
  constexpr int A_PER_T = (A_VECS + kThreads - 1) / kThreads;
  constexpr int A_VPR = BK / 8;                       // vectors per A row
  constexpr int BNK_VECS = BN * BK / 8;
  constexpr int BNK_PER_T = (BNK_VECS + kThreads - 1) / kThreads;
  constexpr int BKN_ITEMS = (BK / 2) * (BN / 8);      // (k-pair, 8 columns)
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

  // ---- main loop ----
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

  // ---- split-K: exchange partial tiles, last arrival reduces ----
  if (numSlices > 1) {
    __shared__ uint32_t sArrival;
    constexpr int ACC_V4 = MI * NI * 4; // float4 vectors per thread
    float4v *ws = reinterpret_cast<float4v *>(p.workspace) +
                  (int64_t(tile) * numSlices) * (ACC_V4 * kThreads);
    {
      float4v *mine = ws + int64_t(slice) * (ACC_V4 * kThreads);
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
            mine[((i * NI + j) * 4 + g) * kThreads + tid] = v;
          }
    }
    __threadfence();
    __syncthreads();
    if (tid == 0)
      sArrival = __hip_atomic_fetch_add(&p.counters[tile], 1u,
                                        __ATOMIC_ACQ_REL,
                                        __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (sArrival != uint32_t(numSlices - 1))
      return; // uniform across the workgroup
    __threadfence();
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int j = 0; j < NI; j++)
#pragma unroll
        for (int e = 0; e < 16; e++)
          acc[i][j][e] = 0.f;
    for (int s = 0; s < numSlices; s++) {
      const float4v *part = ws + int64_t(s) * (ACC_V4 * kThreads);
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            const float4v v = __builtin_nontemporal_load(
                &part[((i * NI + j) * 4 + g) * kThreads + tid]);
#pragma unroll
            for (int e = 0; e < 4; e++)
              acc[i][j][g * 4 + e] += v[e];
          }
    }
    if (tid == 0)
      __hip_atomic_store(&p.counters[tile], 0u, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- epilogue ----
  // Transposed MFMA block: accumulator e of lane l is
  //   column n = 8*(e/4) + 4*(l/32) + e%4,  row m = l%32   (within the block).
  const int l32 = lane % 32, kb = lane / 32;
  const bool useC = p.beta != 0.f;
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
        if (VEC == 8) {
          if (n >= p.N)
            continue;
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

// ------------------------------------------------------------ kernel table --
template <int BM, int BN, int BK, int WM, int WN, int EPI, bool B_NK, int VEC>
Status launchInstance(const GemmProblem &pr, hipStream_t s) {
  constexpr int kThreads = WM * WN * kWave;
  constexpr int A_LD = BK + 8, BP_LD = BN + 8;
  constexpr int A_BYTES = BM * A_LD * 2;
  constexpr int B_BYTES = B_NK ? BN * A_LD * 2 : (BK / 2) * BP_LD * 4;
  constexpr int SMEM = 2 * (A_BYTES + B_BYTES);

  GemmParams p;
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
  p.tilesM = int((pr.M + BM - 1) / BM);
  p.tilesN = int((pr.N + BN - 1) / BN);
  const int kTiles = int((pr.K + BK - 1) / BK);
  int splitK = pr.splitK < 1 ? 1 : pr.splitK;
  if (splitK > kTiles)
    splitK = kTiles > 0 ? kTiles : 1;
  p.kTilesPerSlice = (kTiles + splitK - 1) / splitK;
  // Drop slices that would be empty after rounding up.
  if (p.kTilesPerSlice > 0)
    splitK = (kTiles + p.kTilesPerSlice - 1) / p.kTilesPerSlice;
  if (splitK < 1)
    splitK = 1;
  const int64_t nTiles = int64_t(p.tilesM) * p.tilesN;
  HOM_CHECK_RET(nTiles < (int64_t(1) << 30), Status::kInvalidArgument,
                "gemm: too many output tiles (%lld)", (long long)nTiles);
  p.workspace = nullptr;
  p.counters = nullptr;
  if (splitK > 1) {
    const size_t wsBytes =
        size_t(nTiles) * splitK * size_t(BM) * BN * sizeof(float);
    p.workspace = static_cast<float *>(scratch(kWorkspace, wsBytes, false));
    p.counters = static_cast<uint32_t *>(
        scratch(kCounters, size_t(nTiles) * sizeof(uint32_t), true));
    if (!p.workspace || !p.counters)
      return Status::kInternal;
  }
  auto kernel = gemmKernel<BM, BN, BK, WM, WN, EPI, B_NK, VEC>;
  static bool attrSet = false;
  if (!attrSet && SMEM > 48 * 1024) {
    HOM_HIP_RET(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    SMEM),
                Status::kInternal);
  }
  attrSet = true;
  if (nTiles == 0)
    return Status::kSuccess;
  kernel<<<dim3((unsigned)nTiles, (unsigned)splitK), dim3(kThreads), SMEM, s>>>(
      p);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

using LaunchFn = Status (*)(const GemmProblem &, hipStream_t);

struct KernelEntry {
  GemmKernelInfo info;
  LaunchFn nn; // B as [K, N]
  LaunchFn nt; // B as [N, K]
};

#define HOM_GEMM_ENTRY(BM, BN, BK, WM, WN, EPI_ENUM, EPI_STR, ACT, VEC)        \
  {                                                                            \
    {"hom_gfx950_mfma_f16_s32x32x16gemm_f16_" #BM "x" #BN "_" #BK "x2_w" #WM   \
     "x" #WN "_nn_align" #VEC "_" EPI_STR,                                     \
     BM, BN, BK, WM, WN, VEC, ACT, EPI_ENUM},                                  \
        launchInstance<BM, BN, BK, WM, WN, int(EPI_ENUM), false, VEC>,         \
        launchInstance<BM, BN, BK, WM, WN, int(EPI_ENUM), true, VEC>           \
  }

#define HOM_GEMM_TILE(BM, BN, BK, WM, WN, VEC)                                 \
  HOM_GEMM_ENTRY(BM, BN, BK, WM, WN, Epilogue::kLinear, "linear", 0, VEC),     \
      HOM_GEMM_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluErf, "gelu", 1, VEC),  \
      HOM_GEMM_ENTRY(BM, BN, BK, WM, WN, Epilogue::kGeluTanh, "gelutanh", 1,   \
                     VEC)

// Manifest order is part of the ABI: compiled modules carry indices into it.
// Append new entries at the end.
const KernelEntry kKernels[] = {
    HOM_GEMM_TILE(128, 128, 32, 2, 2, 8),
    HOM_GEMM_TILE(64, 64, 32, 2, 2, 8),
    HOM_GEMM_TILE(128, 64, 32, 2, 2, 8),
    HOM_GEMM_TILE(64, 128, 32, 2, 2, 8),
    HOM_GEMM_TILE(256, 128, 32, 2, 2, 8),
    HOM_GEMM_TILE(128, 256, 32, 2, 2, 8),
    HOM_GEMM_TILE(128, 128, 64, 2, 2, 8),
    HOM_GEMM_TILE(64, 64, 64, 2, 2, 8),
    HOM_GEMM_TILE(64, 64, 32, 2, 2, 1),
};
constexpr int kNumKernels = sizeof(kKernels) / sizeof(kKernels[0]);

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
    const bool ok = p.N % 8 == 0 && p.K % 8 == 0 && p.lda % 8 == 0 &&
                    p.ldb % 8 == 0 && p.ldd % 4 == 0 &&
                    (p.beta == 0.f || p.ldc % 4 == 0) && aligned16(p.A) &&
                    aligned16(p.B) && aligned16(p.D) &&
                    (p.beta == 0.f || aligned16(p.C));
    HOM_CHECK_RET(ok, Status::kInvalidArgument,
                  "gemm: kernel %s needs N, K and leading dimensions that are "
                  "multiples of 8 and 16-byte aligned operands (M=%lld N=%lld "
                  "K=%lld)",
                  k.info.name, (long long)p.M, (long long)p.N, (long long)p.K);
  }
  if (p.M == 0 || p.N == 0)
    return Status::kSuccess;
  return (p.bIsNK ? k.nt : k.nn)(p, s);
}

} // namespace hom
