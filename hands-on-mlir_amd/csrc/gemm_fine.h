#pragma once

#include "gemm_device.h"

namespace hom {
namespace gemmk {

// ==================================================================== fine ==
// The register-staged pipeline of gemm_pipe.h on the 16x16x32 MFMA
// (v_mfma_f32_16x16x32_f16: 64 lanes x 8 halves per operand, 4 fp32
// accumulators per lane), whose tile sides come in steps of 16 instead of 32.
// That is what lets a 1024-row problem of BERT-base be cut into exactly as
// many tiles as the chip has CUs: 128 x 96 for N = 3072 (8 x 32 = 256 tiles,
// against 192 of 128 x 128), 64 x 48 for N = 768 (16 x 16 = 256, against 192 of
// 64 x 64).  Every CU then pulls less through its L1, multiplies less and has
// less epilogue arithmetic, and none idles.
//
// Operand layout of the instruction, issued with the operands swapped so that
// a lane ends with 4 consecutive columns of one row of D: lane l supplies
// row l % 16 and the 8 k values 8 * (l / 16) .. + 7 of its operand's 32-wide k
// step; accumulator r of lane l is D[row l % 16][column 4 * (l / 16) + r] of
// the 16 x 16 block.
//
// LDS: A and a [N, K] B as in gemm_pipe.h (rows of 128 bytes = 64 k, 16-byte
// chunks XOR-permuted by (row >> 1) & 7, fragments are one ds_read_b128).  A
// row-major B tile keeps k as the row: BN * 2 bytes of data per row in 32-byte
// blocks of 16 columns, rows padded to an odd number t of 32-byte blocks with
// t >= BN / 16 + 4, and the blocks of rows with bit 3 of k set stored four
// blocks to the right.  A transposing read (ds_read_b64_tr_b16) of one 16-column
// block touches rows k..k+3 and k+8..k+11 in its first 32 lanes; with t odd the
// first four land in four different 32-byte bank groups and the shift by four
// puts the other four into the remaining ones.
template <int BN> constexpr int fineRowBytesB() {
  int t = BN / 16 + 4;
  if (t % 2 == 0)
    t += 1;
  return t * 32;
}

template <int BM, int BN, bool B_NK> constexpr int fineStageBytes() {
  return BM * 128 + (B_NK ? BN * 128 : 64 * fineRowBytesB<BN>());
}
template <int BM, int BN, int WM, int WN, bool B_NK> constexpr int fineLdsBytes() {
  // two slab buffers + one 16-byte slot per thread for vectors nobody needs
  // (tile sides that do not divide evenly over the threads); the epilogue's
  // strips (wave tile rows x (columns * 4 + 16) bytes per wavefront) reuse it
  constexpr int kMain =
      2 * fineStageBytes<BM, BN, B_NK>() + WM * WN * kWave * 16;
  constexpr int kStrips = BM * WN * ((BN / WN) * 4 + 16);
  return kMain > kStrips ? kMain : kStrips;
}

// Partial tile of one K slice -> workspace, in accumulator order.
template <int MI, int NI, int THREADS>
__device__ __forceinline__ void fineStorePartial(const GemmParams &p,
                                                 float4v (&acc)[MI][NI],
                                                 int tile, int slice,
                                                 int numSlices, int tid) {
  float4v *mine = reinterpret_cast<float4v *>(p.workspace) +
                  (int64_t(tile) * numSlices + slice) * (MI * NI * THREADS);
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
      mine[(i * NI + j) * THREADS + tid] = acc[i][j];
}

// alpha * acc + beta * C, activation, for 4 consecutive columns of one row:
// the general (any source period, edge columns) form of the epilogue.
template <int EPI>
__device__ __forceinline__ void fineStoreQuad(const GemmParams &p,
                                              const float4v &acc, int m, int n) {
  if (m >= p.M || n >= p.N)
    return;
  const bool useC = p.beta != 0.f;
  const int64_t cRow = int64_t(rowInPeriod(p, m)) * p.ldc;
  const int64_t dRow = int64_t(m) * p.ldd;
  // (N, ldc, ldd are multiples of 8 for these kernels: whole quads)
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
}

// Sums the slices of a split-K launch in slice order and finishes the outputs:
// one thread per accumulator quad of the partial-tile layout.
template <int BM, int BN, int WM, int WN, int EPI>
__global__ __launch_bounds__(256) void fineReduceKernel(GemmParams p,
                                                        int numSlices) {
  constexpr int THREADS = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int MI = WTM / 16, NI = WTN / 16;
  constexpr int PER_TILE = MI * NI * THREADS;
  const int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= int64_t(p.tilesM) * p.tilesN * PER_TILE)
    return;
  const int tile = int(idx / PER_TILE), rem = int(idx % PER_TILE);
  const int q = rem / THREADS, t = rem % THREADS;
  const int i = q / NI, j = q % NI;
  const int lane = t % kWave, wave = t / kWave;
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
    for (int u = 0; u < 4; u++)
      acc += v[u];
  }
  for (; sl < numSlices; sl++)
    acc += part[int64_t(sl) * PER_TILE];
  const int m = tileM * BM + (wave / WN) * WTM + i * 16 + lane % 16;
  const int n = tileN * BN + (wave % WN) * WTN + j * 16 + 4 * (lane / 16);
  fineStoreQuad<EPI>(p, acc, m, n);
}

// The fast epilogue (N, ldc, ldd multiples of 8, 16-byte aligned C and D, a
// source that is absent, one bias row or a full matrix; p.epiMode): the
// wavefront's accumulators go through its private LDS strip (wave tile rows x
// WTN fp32, rows padded by 16 bytes) and leave as 16-byte vectors, WTN / 8 lanes
// per output row, through buffer descriptors based at the wavefront's first
// row (rows past M fall outside; lanes without a vector and columns past N get
// an offset outside).
template <int MI, int NI, int EPI, int CMODE>
__device__ __forceinline__ void
fineEpilogueFast(const GemmParams &p, float4v (&acc)[MI][NI], int rowBase,
                 int colBase, int lane, unsigned char *mine) {
  constexpr int WTM = MI * 16, WTN = NI * 16;
  constexpr int ROW_B = WTN * 4 + 16;
  constexpr int LPR = WTN / 8; // lanes per output row
  constexpr int TOTAL = WTM * LPR;
  constexpr int PASSES = (TOTAL + kWave - 1) / kWave;
  constexpr uint32_t kOob = 0x80000000u;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  auto clampBytes = [](int64_t b) -> int32_t {
    return b > 0x7fffffffLL ? 0x7fffffff : (b < 0 ? 0 : int32_t(b));
  };
  const int rowsLeft = p.M - rowBase;
  const auto rsrcD = __builtin_amdgcn_make_buffer_rsrc(
      p.D + int64_t(rowBase) * p.ldd + colBase, 0,
      clampBytes((int64_t(rowsLeft) * p.ldd - colBase) * 2), 0x00020000);
  const auto rsrcC = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(p.C) + (CMODE == 2 ? int64_t(rowBase) * p.ldc : 0) +
          colBase,
      0,
      CMODE == 2   ? clampBytes((int64_t(rowsLeft) * p.ldc - colBase) * 2)
      : CMODE == 1 ? clampBytes(int64_t(p.N - colBase) * 2)
                   : 0,
      0x00020000);
  const uint32_t ldd2 = uint32_t(p.ldd) * 2u, ldc2 = uint32_t(p.ldc) * 2u;
  // this lane's vectors: index v = pass * 64 + lane -> (row, 8-column group)
  int row[PASSES], col[PASSES];
  bool live[PASSES];
  half8 cv[PASSES];
#pragma unroll
  for (int ps = 0; ps < PASSES; ps++) {
    const int v = ps * kWave + lane;
    row[ps] = v / LPR;
    col[ps] = (v % LPR) * 8;
    live[ps] = (TOTAL % kWave == 0 || v < TOTAL) && colBase + col[ps] < p.N;
    if (!(TOTAL % kWave == 0) && v >= TOTAL)
      row[ps] = 0;
    if constexpr (CMODE != 0) {
      const uint32_t off = (CMODE == 2 ? uint32_t(row[ps]) * ldc2 : 0u) +
                           uint32_t(col[ps]) * 2u;
      cv[ps] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(
                     rsrcC, live[ps] ? off : kOob, 0, 0));
    }
  }
  __syncthreads(); // nobody still reads operands from this LDS
  const int r16 = lane % 16, g = lane / 16;
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
      *reinterpret_cast<float4v *>(mine + (i * 16 + r16) * ROW_B +
                                   (j * 16 + 4 * g) * 4) = acc[i][j];
  float4v lo[PASSES], hi[PASSES];
#pragma unroll
  for (int ps = 0; ps < PASSES; ps++) {
    const unsigned char *src = mine + row[ps] * ROW_B + col[ps] * 4;
    lo[ps] = *reinterpret_cast<const float4v *>(src);
    hi[ps] = *reinterpret_cast<const float4v *>(src + 16);
  }
#pragma unroll
  for (int ps = 0; ps < PASSES; ps++) {
    half8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      float v = p.alpha * (e < 4 ? lo[ps][e] : hi[ps][e - 4]);
      if constexpr (CMODE != 0)
        v = fmaf(p.beta, float(cv[ps][e]), v);
      o[e] = _Float16(activate<EPI>(v));
    }
    __builtin_amdgcn_raw_buffer_store_b128(
        __builtin_bit_cast(u32x4, o), rsrcD,
        live[ps] ? uint32_t(row[ps]) * ldd2 + uint32_t(col[ps]) * 2u : kOob, 0,
        kWriteThroughAux);
  }
}

template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK>
__global__ __launch_bounds__(WM *WN *kWave) void gemmFineKernel(
    const _Float16 *argA, const _Float16 *argB, int argM, int argN, int argK,
    int argLda, int argLdb, int argTilesN, int argXcdQ, uint32_t argTileWalk,
    uint32_t argGroupMagic, int argKTilesPerSlice, GemmParams rest) {
  // Leading scalar arguments arrive in scalar registers with the wavefront;
  // `rest` is read through the kernel-argument pointer behind the first loads
  // (see gemm_pipe.h).
  (void)rest;
  constexpr int kRestOffset = 2 * 8 + 10 * 4;
  static_assert(kRestOffset % alignof(GemmParams) == 0, "argument layout");
  static_assert(DIST >= 1, "at least one slab of global loads in flight");
  constexpr int BK = 64;
  constexpr int THREADS = WM * WN * kWave;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile in steps of 16");
  constexpr int MI = WTM / 16, NI = WTN / 16;
  constexpr int A_BYTES = BM * 128;
  constexpr int SB = fineRowBytesB<BN>(); // row-major B: bytes per k row
  constexpr int B_BYTES = B_NK ? BN * 128 : 64 * SB;
  constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_VECS = BM * 8, B_VECS = BN * 8;
  static_assert(A_VECS % THREADS == 0, "A tile must split evenly over the threads");
  constexpr int A_PER_T = A_VECS / THREADS;
  constexpr int B_PER_T = (B_VECS + THREADS - 1) / THREADS;
  constexpr bool kEvenB = B_VECS % THREADS == 0;
  constexpr int B_VPR = B_NK ? 8 : BN / 8; // vectors per row of the B tile
  constexpr int KSTEPS = BK / 32;
  constexpr int kDummy = 2 * STAGE_BYTES; // per-thread slots for unused vectors
  static_assert((THREADS / 8) % 16 == 0, "vector step must preserve the K swizzle");

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  GemmParams p = {};
  p.A = argA;
  p.B = argB;
  p.M = argM;
  p.N = argN;
  p.K = argK;
  p.lda = argLda;
  p.ldb = argLdb;
  p.tilesN = argTilesN;
  p.xcdQ = argXcdQ;
  p.xcdR = int(argTileWalk & 15u);
  p.lastRows = int((argTileWalk >> 4) & 15u);
  p.fullGroups = int(argTileWalk >> 8);
  p.groupMagic = argGroupMagic;
  p.kTilesPerSlice = argKTilesPerSlice;

  int tid = threadIdx.x;
  int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int waveM = wave / WN, waveN = wave % WN;
  const int l16 = lane % 16, kg = lane / 16;
  int tileM, tileN;
  const int tile = tileCoordsFast(p, blockIdx.x, &tileM, &tileN);
  const int m0 = tileM * BM, n0 = tileN * BN;
  const int slice = blockIdx.y, numSlices = gridDim.y;
  const int kTiles = (p.K + BK - 1) / BK;
  const int ktBegin = slice * p.kTilesPerSlice;
  int ktEnd = ktBegin + p.kTilesPerSlice;
  if (ktEnd > kTiles)
    ktEnd = kTiles;

  // ---- global sources (as in gemm_pipe.h: descriptors based at the tile,
  // rows past the edge read as zero, no branch around a load) ----
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
  int aK[A_PER_T], bK[B_PER_T]; // k position inside the slab
  int aDst0 = 0, bDst[B_PER_T];
  constexpr int DST_STEP = THREADS * 16; // A (and [N, K] B): see gemm_pipe.h
#pragma unroll
  for (int i = 0; i < A_PER_T; i++) {
    const int v = tid + i * THREADS;
    const int r = v / 8, c = v % 8;
    aK[i] = c * 8;
    aOff[i] = (uint32_t(r) * uint32_t(p.lda) + c * 8) * 2u;
    if (i == 0)
      aDst0 = r * 128 + swzK(r, c) * 16;
  }
#pragma unroll
  for (int i = 0; i < B_PER_T; i++) {
    const int v = tid + i * THREADS;
    const bool mine = kEvenB || i + 1 < B_PER_T || v < B_VECS;
    const int r = v / B_VPR, c = v % B_VPR;
    if (B_NK) {
      bK[i] = c * 8;
      bOff[i] = mine ? (uint32_t(r) * uint32_t(p.ldb) + c * 8) * 2u : kOob;
      bDst[i] = mine ? A_BYTES + r * 128 + swzK(r, c) * 16 : kDummy + tid * 16;
    } else {
      bK[i] = r;
      bOff[i] = mine ? (uint32_t(r) * uint32_t(p.ldb) + c * 8) * 2u : kOob;
      bDst[i] = mine ? A_BYTES + r * SB + (c / 2 + 4 * ((r >> 3) & 1)) * 32 +
                           (c % 2) * 16
                     : kDummy + tid * 16;
    }
  }

  half8 regA[DIST][A_PER_T], regB[DIST][B_PER_T];
  const int nkFull = (kEnd - ktBegin * BK) / BK;
  const bool hasTail = kEnd - ktBegin * BK > nkFull * BK;
  const int ktLastFull = ktBegin + nkFull - 1;
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
    unsigned char *st = smem + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < A_PER_T; i++)
      *reinterpret_cast<half8 *>(st + aDst0 + i * DST_STEP) = regA[S][i];
#pragma unroll
    for (int i = 0; i < B_PER_T; i++) {
      // (a slot outside the slab buffers is the same for both stages)
      unsigned char *dst = bDst[i] >= kDummy ? smem + bDst[i] : st + bDst[i];
      *reinterpret_cast<half8 *>(dst) = regB[S][i];
    }
  };

  // The first DIST slabs are requested before anything else is set up.
  if (nkFull > 0) {
    staticFor<DIST>(
        [&](auto d) { loadGlobal(ktBegin + decltype(d)::value, d); });
  }
  __builtin_amdgcn_sched_barrier(0);
#if defined(__HIP_DEVICE_COMPILE__) // (the host pass only needs the kernel's stub)
  {
    typedef const __attribute__((address_space(4))) GemmParams *RestPtr;
    RestPtr late = (RestPtr)(
        (const __attribute__((address_space(4))) char *)
            __builtin_amdgcn_kernarg_segment_ptr() +
        kRestOffset);
    p = *late;
  }
#endif

  float4v acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
      acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // ---- fragment addresses ----
  // Rows of a wavefront start at multiples of 16, so the swizzle term
  // (row >> 1) & 7 only involves the lane's row inside the block.
  const int swzLane = (l16 >> 1) & 7;
  int aFrag[KSTEPS], bFragK[KSTEPS];
#pragma unroll
  for (int kk = 0; kk < KSTEPS; kk++) {
    aFrag[kk] = (waveM * WTM + l16) * 128 + ((kk * 4 + kg) ^ swzLane) * 16;
    bFragK[kk] =
        A_BYTES + (waveN * WTN + l16) * 128 + ((kk * 4 + kg) ^ swzLane) * 16;
  }
  // Row-major B, transposing reads: source lane L = lane % 16 of a 16-lane
  // group supplies row kbase + L / 4 and the 4 columns at (L % 4) * 4 of the
  // block's 16; the group's k rows are 8 * kg + 4 * h + L / 4 for the two
  // reads h = 0, 1 of a k step, so bit 3 of k is kg & 1.
  const int trRow = l16 / 4, trCol = (l16 % 4) * 4;
  const int bFragN = A_BYTES + (kg * 8 + trRow) * SB + 4 * (kg & 1) * 32 +
                     (waveN * WTN) * 2 + trCol * 2;

  auto loadFragUnit = [&](int stage, int kk, half8 (&fa)[MI], half8 (&fb)[NI],
                          auto uC) {
    constexpr int U = decltype(uC)::value;
    const unsigned char *st = smem + stage * STAGE_BYTES;
    if constexpr (U < MI) {
      fa[U] = *reinterpret_cast<const half8 *>(st + aFrag[kk] + U * 16 * 128);
    } else if constexpr (B_NK) {
      constexpr int j = U - MI;
      fb[j] = *reinterpret_cast<const half8 *>(st + bFragK[kk] + j * 16 * 128);
    } else {
      constexpr int j = U - MI;
      short4v t[2];
#pragma unroll
      for (int h = 0; h < 2; h++)
        t[h] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) short4v *)(
                st + bFragN + (kk * 32 + h * 4) * SB + j * 32));
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

  // ---- main loop: the scheme of gemm_pipe.h with two 32-wide k steps ----
  constexpr int NV = A_PER_T + B_PER_T;
  constexpr int NM = MI * NI;
  half8 fa[2][MI], fb[2][NI];
  const int nk = nkFull;
  auto stageVec = [&](int stage, int kt, auto setC, auto vC) {
    constexpr int S = decltype(setC)::value;
    constexpr int V = decltype(vC)::value;
    unsigned char *st = smem + stage * STAGE_BYTES;
    const int k0 = kt * BK;
    if constexpr (V < A_PER_T) {
      *reinterpret_cast<half8 *>(st + aDst0 + V * DST_STEP) = regA[S][V];
      regA[S][V] = __builtin_bit_cast(
          half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcA, aOff[V],
                                                       uint32_t(k0) * 2u, 0));
    } else {
      constexpr int W = V - A_PER_T;
      unsigned char *dst = bDst[W] >= kDummy ? smem + bDst[W] : st + bDst[W];
      *reinterpret_cast<half8 *>(dst) = regB[S][W];
      regB[S][W] = __builtin_bit_cast(
          half8,
          __builtin_amdgcn_raw_buffer_load_b128(
              rsrcB, bOff[W],
              B_NK ? uint32_t(k0) * 2u : uint32_t(k0) * uint32_t(p.ldb) * 2u,
              0));
    }
  };
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
      acc[m / NI][m % NI] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
          b[m % NI], a[m / NI], acc[m / NI][m % NI], 0, 0, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  auto slab = [&](int i, auto setC, auto tailC) {
    constexpr bool kTail = decltype(tailC)::value;
    const int cur = i & 1;
    const bool more = !kTail || i + 1 < nk;
    const int ktWant = ktBegin + i + 1 + DIST;
    const int ktNext = ktWant < ktLastFull ? ktWant : ktLastFull;
    using V0C = std::integral_constant<int, 0>;
    using V1C = std::integral_constant<int, NV>;
    // k step 0: multiplies, moves slab i+1 to the other buffer, fetches the
    // fragments of k step 1
    mfmaMixed(fa[0], fb[0], fa[1], fb[1], cur, 1, std::true_type{}, cur ^ 1,
              ktNext, more, setC, V0C{}, V1C{});
    // k step 1, behind the barrier that completes slab i+1: multiplies and
    // fetches the first fragments of slab i+1
    if (more) {
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      mfmaMixed(fa[1], fb[1], fa[0], fb[0], cur ^ 1, 0, std::true_type{}, 0, 0,
                false, setC, V1C{}, V1C{});
    } else {
      mfmaMixed(fa[1], fb[1], fa[0], fb[0], 0, 0, std::false_type{}, 0, 0,
                false, setC, V1C{}, V1C{});
    }
  };
  if (nk > 0) {
    storeLds(0, std::integral_constant<int, 0>{});
    loadGlobal(ktBegin + DIST, std::integral_constant<int, 0>{});
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    loadFrags(0, 0, fa[0], fb[0]);
    int i = 0;
    for (; i + DIST < nk; i += DIST) {
      staticFor<DIST>([&](auto d) {
        constexpr int Dd = decltype(d)::value;
        slab(i + Dd, std::integral_constant<int, (Dd + 1) % DIST>{},
             std::false_type{});
      });
    }
    bool go = true;
    staticFor<DIST>([&](auto d) {
      constexpr int Dd = decltype(d)::value;
      go = go && i + Dd < nk;
      if (go)
        slab(i + Dd, std::integral_constant<int, (Dd + 1) % DIST>{},
             std::true_type{});
    });
  }
  if (hasTail) {
    // The partial slab of a ragged K, unpipelined, behind the full ones.
    using Set0 = std::integral_constant<int, 0>;
    loadGlobalChecked(ktBegin + nkFull, Set0{});
    __syncthreads(); // no wavefront still reads a full slab from buffer 0
    storeLds(0, Set0{});
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KSTEPS; kk++) {
      loadFrags(0, kk, fa[0], fb[0]);
#pragma unroll
      for (int m = 0; m < NM; m++)
        acc[m / NI][m % NI] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            fb[0][m % NI], fa[0][m / NI], acc[m / NI][m % NI], 0, 0, 0);
    }
  }

  if (numSlices > 1) {
    fineStorePartial<MI, NI, THREADS>(p, acc, tile, slice, numSlices, tid);
    return;
  }
  const int rowBase = m0 + waveM * WTM, colBase = n0 + waveN * WTN;
  if constexpr (EPI <= int(Epilogue::kGeluTanh)) {
    unsigned char *mine = smem + wave * (WTM * (WTN * 4 + 16));
    const int mode = p.epiMode;
    if (mode == 0)
      return fineEpilogueFast<MI, NI, EPI, 0>(p, acc, rowBase, colBase, lane, mine);
    if (mode == 1)
      return fineEpilogueFast<MI, NI, EPI, 1>(p, acc, rowBase, colBase, lane, mine);
    if (mode == 2)
      return fineEpilogueFast<MI, NI, EPI, 2>(p, acc, rowBase, colBase, lane, mine);
  }
  // general form: the lane's quads where the accumulators are
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < NI; j++)
      fineStoreQuad<EPI>(p, acc[i][j], rowBase + i * 16 + l16,
                         colBase + j * 16 + 4 * kg);
}

template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK>
Status launchFine(const GemmProblem &pr, hipStream_t s) {
  constexpr int SMEM = fineLdsBytes<BM, BN, WM, WN, B_NK>();
  static_assert(SMEM <= 160 * 1024, "LDS");
  LaunchPlan plan;
  Status st = planLaunch<BM, BN, 64>(pr, &plan);
  if (st != Status::kSuccess)
    return st;
  HOM_CHECK_RET(B_NK || pr.K * pr.ldb * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument,
                "gemm: B larger than 2 GiB is not supported by this kernel");
  HOM_CHECK_RET((int64_t(BM) * pr.lda + pr.K) * 2 < (int64_t(1) << 31) &&
                    (int64_t(BN) * pr.ldb + pr.K) * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument, "gemm: leading dimension too large");
  auto kernel = gemmFineKernel<BM, BN, WM, WN, DIST, EPI, B_NK>;
  static bool attrSet = false;
  st = allowLds(kernel, SMEM, &attrSet);
  if (st != Status::kSuccess)
    return st;
  if (plan.nTiles == 0)
    return Status::kSuccess;
  const GemmParams &q = plan.p;
  kernel<<<dim3((unsigned)plan.nTiles, (unsigned)plan.splitK),
           dim3(WM * WN * kWave), SMEM, s>>>(
      q.A, q.B, q.M, q.N, q.K, int(q.lda), int(q.ldb), q.tilesN, q.xcdQ,
      uint32_t(q.xcdR) | uint32_t(q.lastRows) << 4 | uint32_t(q.fullGroups) << 8,
      q.groupMagic, q.kTilesPerSlice, q);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  if (plan.splitK > 1) {
    constexpr int kPerTile = (BM / 16) * (BN / 16) * kWave;
    const int64_t groups = plan.nTiles * kPerTile;
    fineReduceKernel<BM, BN, WM, WN, EPI>
        <<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s>>>(
            plan.p, plan.splitK);
    HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  }
  return Status::kSuccess;
}

} // namespace gemmk
} // namespace hom
