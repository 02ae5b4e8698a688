// "staged" kernels (any shape / alignment, and the bring-up path): global ->
// registers -> LDS with two LDS buffers and padded LDS rows; row-major B is
// interleaved into (k, k+1) half2 pairs while it is staged.
#pragma once

#include "gemm_device.h"

namespace hom {
namespace gemmk {

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

} // namespace gemmk
} // namespace hom
