#pragma once

#include "gemm_device.h"

namespace hom {
namespace gemmk {

// ==================================================================== pipe ==
// Same LDS layout, fragment reads and barrier placement as the dma kernels.
// DMA == false: the slabs travel global -> registers -> LDS (two LDS buffers);
// the loads of slab i+1 are issued before slab i is multiplied and written to
// LDS after it, DIST slabs are in flight in registers.  DMA == true: the same
// pipeline with buffer_load ... lds into a ring of DIST + 1 LDS buffers, which
// takes the staging writes (75 bytes per clock and CU when issued from
// registers, a third of the read rate) off the LDS pipe the fragment reads
// need.  Both stage at the rate the L1 delivers (about 50 bytes per clock and
// CU); the DMA variant is 1.5-8 % faster at M = 1024 and equal for 256 x 256
// tiles, where only one slab in flight fits in LDS.
// What the kernel needs on its way to the first loads travels as leading
// scalar arguments (14 dwords): the command processor delivers those in scalar
// registers when the wavefront starts (kernel-argument preload, see the
// Makefile), so the first requests do not wait for an argument fetch from
// memory.  `rest` holds the same values again plus everything else; its copies
// of the leading arguments are never read.
// tileWalk = xcdR | lastRows << 4 | fullGroups << 8.
template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK,
          bool DMA = false>
__global__ __launch_bounds__(WM *WN *kWave) void gemmPipeKernel(
    const _Float16 *argA, const _Float16 *argB, int argM, int argN, int argK,
    int argLda, int argLdb, int argTilesN, int argXcdQ, uint32_t argTileWalk,
    uint32_t argGroupMagic, int argKTilesPerSlice, GemmParams rest) {
  // `rest` is read through the kernel-argument pointer, per tile and behind the
  // first loads (see below): named here, it would be fetched - and waited for
  // - ahead of everything.
  (void)rest;
  constexpr int kRestOffset = 2 * 8 + 10 * 4; // bytes of the leading arguments
  static_assert(kRestOffset % alignof(GemmParams) == 0, "argument layout");
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
  // DMA: slabs travel global memory -> LDS without passing through registers
  // (buffer_load ... lds), into a ring of DIST + 1 buffers: the slab being
  // multiplied and DIST slabs landed or on their way.  An LDS write from
  // registers moves 75 bytes per clock and CU and takes the LDS pipe from the
  // fragment reads; the DMA path leaves it to them.
  constexpr int NBUF = DMA ? DIST + 1 : 2;
  // Tiles up to 128 x 128 serve problems of a few microseconds, where the way
  // to the first memory request and back counts as much as the main loop;
  // larger tiles keep the order that suits their register budget.
  constexpr bool kLatencyFirst = BM * BN <= 128 * 128;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  // The wavefront index is the same for every lane; saying so keeps what is
  // derived from it (the wavefront's rows and columns, the descriptors of its
  // output rows) in scalar registers.
  const int tid0 = threadIdx.x;
  const int wave0 = __builtin_amdgcn_readfirstlane(tid0 / kWave);

  // Persistent over tiles: the grid holds at most as many workgroups as fit on
  // the chip at once and each walks tiles pid, pid + grid, ...  (the grid is a
  // multiple of the XCD count, so a workgroup's tiles stay in its XCD's
  // contiguous range).  A tile's output stores drain and the next tile's first
  // slabs arrive while other work runs, instead of between two workgroups.
  // The grid never holds more workgroups than there are tiles, so the first
  // tile needs no test (a test ahead of everything would make the kernel wait
  // for two kernel-argument fetches in a row).
  int vpid = blockIdx.x;
  int nTiles;
  do {
  if (vpid != int(blockIdx.x))
    __syncthreads(); // the previous tile's epilogue strips live in this LDS
  // Small tiles (kLatencyFirst): what the tile loop would let the compiler
  // compute once, ahead of the first tile's loads (fragment addresses, the
  // epilogue's descriptors), is tied to these two values, which it must take
  // as new in every round: a kernel that runs a few microseconds cannot afford
  // a microsecond of set-up in front of its first memory request.
  int tid = tid0, wave = wave0;
  if constexpr (kLatencyFirst)
    asm volatile("" : "+v"(tid), "+s"(wave));
  const int lane = tid % kWave;
  const int waveM = wave / WN, waveN = wave % WN;
  const int l32 = lane % 32, kb = lane / 32;
  int tileM, tileN;
  const int tile = tileCoordsFast(p, vpid, &tileM, &tileN);
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
  // scalar offset per slab.  Rows past the edge (of A, of B given as [N, K])
  // fall outside the descriptor and read as zero; columns of a row-major B past
  // the edge read whatever follows in memory (the next row, or zero past the
  // tensor): what they fetch only reaches outputs that are never stored.
  // Every slab issues the same number of loads and there is no branch
  // around a load, so the compiler's outstanding-load counts are exact (a
  // branch makes it wait for everything in flight and defeats the pipeline).
  // The main loop walks the slice's FULL slabs only and asks for no range
  // test per vector: vector instructions in that loop cost matrix-core time.
  // A slab requested past the last full one is replaced by the last full one
  // (it is never used), and a partial last slab (K not a multiple of 64) is
  // multiplied behind the loop by a short unpipelined pass whose loads map
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
  // (a 96-column row-major B tile is stored without a swizzle: its vectors lie
  // in LDS in the order of their index)
  static_assert((THREADS / 8) % 16 == 0 &&
                    (B_NK || BN == 96 ||
                     (THREADS % B_VPR == 0 && (THREADS / B_VPR) % 4 == 0)),
                "vector step must preserve the LDS swizzles");
  int aDst0 = 0, bDst0 = 0;
  int aK[A_PER_T], bK[B_PER_T]; // k position inside the slab
#pragma unroll
  // DMA: a wavefront's instruction fills 1 KiB of LDS in lane order, so vector v
  // lands at byte 16 v and the swizzle is applied on the source side: the lane
  // fetches the chunk that belongs at its position.
  for (int i = 0; i < A_PER_T; i++) {
    const int v = tid + i * THREADS;
    const int r = v / 8, c = DMA ? swzK(r, v % 8) : v % 8;
    aK[i] = c * 8;
    aOff[i] = (uint32_t(r) * uint32_t(p.lda) + c * 8) * 2u;
    if (i == 0)
      aDst0 = DMA ? v * 16 : r * 128 + swzK(r, c) * 16;
  }
#pragma unroll
  for (int i = 0; i < B_PER_T; i++) {
    const int v = tid + i * THREADS;
    const int r = v / B_VPR, pc = v % B_VPR;
    if (B_NK) {
      const int c = DMA ? swzK(r, pc) : pc;
      bK[i] = c * 8;
      bOff[i] = (uint32_t(r) * uint32_t(p.ldb) + c * 8) * 2u;
      if (i == 0)
        bDst0 = DMA ? v * 16 : r * 128 + swzK(r, c) * 16;
    } else {
      const int c = DMA ? swzN<BN>(r, pc / 4) * 4 + pc % 4 : pc;
      bK[i] = r;
      bOff[i] = (uint32_t(r) * uint32_t(p.ldb) + c * 8) * 2u;
      if (i == 0)
        bDst0 = DMA ? v * 16
                    : r * B_ROW_BYTES + swzN<BN>(r, c / 4) * 64 + (c % 4) * 16;
    }
  }

  half8 regA[DMA ? 1 : DIST][A_PER_T], regB[DMA ? 1 : DIST][B_PER_T];
  // Slabs of this slice that lie inside [0, kEnd) entirely, and whether a
  // partial one follows them (only the last slice of a ragged K has one).
  const int nkFull = (kEnd - ktBegin * BK) / BK;
  const bool hasTail = kEnd - ktBegin * BK > nkFull * BK;
  const int ktLastFull = ktBegin + nkFull - 1;
  // Full slab kt (requests past the last full slab fetch that one again).
  // One vector of a full slab straight into LDS buffer `stage` (DMA).
  auto dmaVec = [&](int stage, int k0, auto vC) {
#if defined(__HIP_DEVICE_COMPILE__) // (the builtin's LDS pointer type exists only for the GPU target)
    constexpr int V = decltype(vC)::value;
    unsigned char *st = smem + stage * STAGE_BYTES;
    if constexpr (V < A_PER_T) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrcA, HOM_LDS_PTR(st + (V * THREADS + wave * kWave) * 16), 16,
          aOff[V], uint32_t(k0) * 2u, 0, 0);
    } else {
      constexpr int W = V - A_PER_T;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          rsrcB, HOM_LDS_PTR(st + A_BYTES + (W * THREADS + wave * kWave) * 16),
          16, bOff[W],
          B_NK ? uint32_t(k0) * 2u : uint32_t(k0) * uint32_t(p.ldb) * 2u, 0, 0);
    }
#endif
  };
  auto loadGlobal = [&](int kt, auto setC) {
    constexpr int S = decltype(setC)::value;
    const int k0 = (kt < ktLastFull ? kt : ktLastFull) * BK;
    if constexpr (DMA) {
      // (set S: the slab goes to ring buffer S)
      staticFor<A_PER_T + B_PER_T>([&](auto vC) { dmaVec(S, k0, vC); });
    } else {
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
    }
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

  // The first DIST slabs are requested before anything else is set up.
  // Small tiles: the first DIST slabs are requested before anything else is
  // set up.
  if constexpr (kLatencyFirst) {
    if (nkFull > 0) {
      staticFor<DIST>(
          [&](auto d) { loadGlobal(ktBegin + decltype(d)::value, d); });
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // Everything else the kernel was given.  The pointer is made opaque so that
  // these fetches (and what is derived from them: the epilogue's descriptors
  // and range tests) stay here, behind the first loads, in every round.
#if defined(__HIP_DEVICE_COMPILE__) // (the host pass only needs the kernel's stub)
  {
    typedef const __attribute__((address_space(4))) GemmParams *RestPtr;
    RestPtr late = (RestPtr)(
        (const __attribute__((address_space(4))) char *)
            __builtin_amdgcn_kernarg_segment_ptr() +
        kRestOffset);
    if constexpr (kLatencyFirst)
      asm volatile("" : "+s"(late));
    p = *late;
  }
#endif
  nTiles = p.tilesM * p.tilesN;
  // Folded layer norm: the partial sums of this thread's row are requested
  // next to the first slabs.  Tiles of 128 rows and more, which have few
  // registers to spare, reduce them before the main loop starts (two registers
  // live through it, the round trip overlaps the wait for the first slab);
  // 64-row tiles keep the raw pairs until the epilogue, so their main loop does
  // not wait for them (1024 x 768 x 3072: 13.1 -> 12.5 us; the same on 128-row
  // tiles costs 32 registers and 0.5 us).
  constexpr bool kFoldEarly = BM >= 128;
  float2v foldRaw[EPI >= kEpiFoldA ? FoldBatch<BM>::value : 1];
  float2v foldStat{1.f, 0.f};
  if constexpr (EPI >= kEpiFoldA) {
    foldRowStatRequest<BM>(p, m0, tid, foldRaw);
    if constexpr (kFoldEarly) {
      foldStat = foldRowStatFinish<BM>(p, m0, tid, foldRaw);
      asm volatile("" : "+v"(foldStat[0]), "+v"(foldStat[1]));
    }
  }

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

  // Fragment registers: one set per k step parity, or one per k step of a slab
  // (kWholeSlabFrags, see the main loop).  DMA with a row-major B keeps the two
  // halves of a transposed fragment apart until tieFragments() has waited for
  // them.
  constexpr bool kWholeSlabFrags = MI * NI == 1;
  constexpr int FSETS = kWholeSlabFrags ? KSTEPS : 2;
  half8 fa[FSETS][MI], fb[FSETS][NI];
  constexpr bool kHandReads = DMA && !B_NK;
  half8(*const fbSets)[NI] = fb;
  short4v fbHalf[DMA && !B_NK ? FSETS : 1][NI][2];
  // One fragment per call: unit u < MI is A block u, the rest are B blocks.
  auto loadFragUnit = [&](int stage, int kk, half8 (&fa)[MI], half8 (&fb)[NI],
                          auto uC) {
    constexpr int U = decltype(uC)::value;
    const unsigned char *st = smem + stage * STAGE_BYTES;
    if constexpr (U < MI && kHandReads) {
      // (see the B units below: in this mode every fragment read is issued
      // and waited for by hand, so that the waits can be exact)
      // INVARIANT: the registers an asm read writes are not valid until
      // tieFragments() has waited for them; nothing may use or copy fa / fbHalf
      // between the read and that call (the compiler believes they are ready).
      const uint32_t at = uint32_t(uintptr_t(HOM_LDS_PTR(st + aFrag[kk])));
      half8 frag;
      asm volatile("ds_read_b128 %0, %1 offset:%2"
                   : "=v"(frag)
                   : "v"(at), "i"(U * 32 * 128));
      fa[U] = frag;
    } else if constexpr (U < MI) {
      fa[U] = *reinterpret_cast<const half8 *>(st + aFrag[kk] + U * 32 * 128);
    } else if constexpr (B_NK) {
      constexpr int j = U - MI;
      fb[j] = *reinterpret_cast<const half8 *>(st + bFragK[kk] + j * 32 * 128);
    } else {
      constexpr int j = U - MI;
      if constexpr (DMA) {
        // Issued behind the compiler's back: it would put a wait for every
        // outstanding DMA load in front of a transposing read (it cannot tell
        // that the read's buffer is not one a load is filling).  The compiler
        // does not count reads it cannot see, so its waits for the reads it
        // can see would come out stricter than needed; hence all of them by
        // hand.  The halves are put together, behind a wait, by
        // tieFragments().
        const int set = int(&fb - fbSets);
        const uint32_t at = uint32_t(uintptr_t(HOM_LDS_PTR(st + bFragN[j])));
#pragma unroll
        for (int h = 0; h < 2; h++) {
          short4v half;
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
                       : "=v"(half)
                       : "v"(at), "i"((kk * 16 + h * 4) * B_ROW_BYTES));
          fbHalf[set][j][h] = half;
        }
      } else {
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
  // Wave tiles of one MFMA block (64x64 with 2x2 wavefronts) keep the fragments
  // of all four k steps of a slab in registers: with a fragment set per k step
  // parity, every k step is one LDS round trip for 32 clocks of MFMA.  With all
  // of a slab's fragments requested at once behind the barrier, a slab exposes
  // one round trip: 1024x768x3072 13.4 -> 12.7 us, 1024x768x768 5.5 -> 5.3 us.
  // (Two blocks per wave tile, 128x128 with 2x4 wavefronts: 2 % slower.)
  const int nk = nkFull; // the pipelined loop walks the full slabs
  // Moves vector v of register set S to LDS and refills it from full slab kt
  // (already clamped to the last full slab by the caller).
  auto stageVec = [&](int stage, int kt, auto setC, auto vC) {
    constexpr int S = decltype(setC)::value;
    constexpr int V = decltype(vC)::value;
    unsigned char *sA = smem + stage * STAGE_BYTES;
    unsigned char *sB = sA + A_BYTES;
    const int k0 = kt * BK;
    if constexpr (DMA) {
      dmaVec(stage, k0, vC);
    } else if constexpr (V < A_PER_T) {
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
  // Row-major B staged by DMA: the transposing reads were issued by hand, so
  // the wait for them is by hand as well, and the fragments pass through it so
  // that no MFMA on them can be moved in front of it.
  // Hand-issued fragment reads (kHandReads): the wait for the fragments of a k
  // step, and the fragments pass through it so that no MFMA on them can be
  // moved in front of it.  allowC: how many LDS reads were issued after the
  // last one of this k step (they may stay outstanding; LDS reads return in
  // order); negative: the caller has waited.
  using TieNow = std::integral_constant<int, 0>;
  auto tieFragments = [&](half8 (&a)[MI], half8 (&b)[NI], auto allowC) {
    constexpr int kAllow = decltype(allowC)::value;
    if constexpr (kHandReads) {
      const int set = int(&b - fbSets);
      if constexpr (kAllow >= 0)
        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kAllow < 15 ? kAllow : 15)
                     : "memory");
      staticFor<MI>([&](auto iC) {
        half8 frag = a[decltype(iC)::value];
        asm volatile("" : "+v"(frag)); // not before the wait
        a[decltype(iC)::value] = frag;
      });
      staticFor<NI>([&](auto jC) {
        constexpr int j = decltype(jC)::value;
        short4v lo = fbHalf[set][j][0], hi = fbHalf[set][j][1];
        asm volatile("" : "+v"(lo), "+v"(hi)); // not before the wait
        typedef short short8v __attribute__((ext_vector_type(8)));
        short8v both;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          both[e] = lo[e];
          both[4 + e] = hi[e];
        }
        b[j] = __builtin_bit_cast(half8, both);
      });
    }
  };
  // The MFMAs of one k step on fragments (a, b).  Spread between them: the
  // fragment reads of another k step (rdStage, rdKk) into (na, nb) when RD, and
  // the staging vectors [V0, V1) when stageOn.  Memory operation q of n goes in
  // front of MFMA q * NM / n.
  auto mfmaMixed = [&](half8 (&a)[MI], half8 (&b)[NI], half8 (&na)[MI],
                       half8 (&nb)[NI], int rdStage, int rdKk, auto rdC,
                       int stStage, int kt, bool stageOn, auto setC, auto v0C,
                       auto v1C, auto allowC) {
    constexpr bool RD = decltype(rdC)::value;
    constexpr int V0 = decltype(v0C)::value, V1 = decltype(v1C)::value;
    constexpr int NR = RD ? MI + NI : 0;
    constexpr int N = NR + (V1 - V0);
    tieFragments(a, b, allowC);
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
  // The barrier between slab i and slab i+1: every wavefront has its last
  // fragments of slab i, and slab i+1 is complete in its buffer.  DMA: a
  // wavefront's loads land in the order it issued them, NV per slab, and slabs
  // up to i+DIST have been issued, so slab i+1 is there when at most
  // (DIST-1) * NV loads are outstanding.
  auto slabBarrier = [&]() {
    if constexpr (DMA)
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(
                       (DIST - 1) * NV)
                   : "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };
  // tailC: the slab may be the last one (then nothing follows it); the
  // steady-state loop knows it is not and runs without branches.
  auto slab = [&](int i, auto setC, auto tailC) {
    constexpr bool kTail = decltype(tailC)::value;
    // Register staging: slab i+1 moves from its registers to the other buffer
    // and the registers are refilled with slab i+1+DIST.  DMA: the buffer that
    // slab i-1 left takes slab i+DIST.
    const int cur = DMA ? i % NBUF : i & 1;
    const int nxt = DMA ? (i + 1) % NBUF : cur ^ 1;
    const int fill = DMA ? (i + DIST) % NBUF : cur ^ 1;
    const bool more = !kTail || i + 1 < nk;
    const int ktWant = ktBegin + i + DIST + (DMA ? 0 : 1);
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
                  fill, ktNext, more, setC, V0C{}, V1C{}, TieNow{});
      } else {
        static_assert(ns == 0, "the next slab finds its first fragments in set 0");
        if (more) {
          // Every wavefront has its last fragments of slab i in registers and
          // slab i+1 is complete in the other buffer after this barrier; its
          // first fragments arrive under the MFMAs of the last k step.
          slabBarrier();
          mfmaMixed(fa[cs], fb[cs], fa[ns], fb[ns], nxt, 0, std::true_type{},
                    0, 0, false, setC, V0C{}, V1C{}, TieNow{});
        } else {
          mfmaMixed(fa[cs], fb[cs], fa[ns], fb[ns], 0, 0, std::false_type{}, 0,
                    0, false, setC, V0C{}, V1C{}, TieNow{});
        }
      }
    });
  };
  // The same slab with every k step's fragments in a register set of its own
  // (kWholeSlabFrags).  On entry the fragments of slab i are in flight or
  // there.  The first KSTEPS-1 k steps carry the staging of slab i+1; behind the
  // barrier that completes it the fragments of its first KSTEPS-1 k steps are
  // requested (their sets are free), the last k step of slab i is multiplied,
  // and the last set is requested again.
  auto slabWhole = [&](int i, auto setC, auto tailC) {
    constexpr bool kTail = decltype(tailC)::value;
    const int cur = DMA ? i % NBUF : i & 1;
    const int nxt = DMA ? (i + 1) % NBUF : cur ^ 1;
    const int fill = DMA ? (i + DIST) % NBUF : cur ^ 1;
    const bool more = !kTail || i + 1 < nk;
    const int ktWant = ktBegin + i + DIST + (DMA ? 0 : 1);
    const int ktNext = ktWant < ktLastFull ? ktWant : ktLastFull;
    staticFor<KSTEPS - 1>([&](auto kkC) {
      constexpr int kk = decltype(kkC)::value;
      constexpr int V0 = kk * NV / ST_STEPS, V1 = (kk + 1) * NV / ST_STEPS;
      using V0C = std::integral_constant<int, V0>;
      using V1C = std::integral_constant<int, V1>;
      constexpr int fs = kk % FSETS;
      // the fragments of the later k steps were requested behind these
      mfmaMixed(fa[fs], fb[fs], fa[fs], fb[fs], 0, 0, std::false_type{},
                fill, ktNext, more, setC, V0C{}, V1C{},
                std::integral_constant<int, (KSTEPS - 1 - kk) *
                                                (MI + 2 * NI)>{});
    });
    constexpr int last = (KSTEPS - 1) % FSETS;
    using VE = std::integral_constant<int, NV>;
    if (more) {
      slabBarrier();
      staticFor<KSTEPS - 1>([&](auto kkC) {
        constexpr int kk = decltype(kkC)::value;
        loadFrags(nxt, kk, fa[kk % FSETS], fb[kk % FSETS]);
      });
      __builtin_amdgcn_sched_barrier(0);
      // the barrier's wait covered the last k step's fragments
      tieFragments(fa[last], fb[last], std::integral_constant<int, 15>{});
    } else {
      tieFragments(fa[last], fb[last], TieNow{});
    }
    mfmaMixed(fa[last], fb[last], fa[last], fb[last], 0, 0, std::false_type{},
              0, 0, false, setC, VE{}, VE{}, std::integral_constant<int, -1>{});
    if (more) {
      loadFrags(nxt, KSTEPS - 1, fa[last], fb[last]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // The partial slab of a ragged K, unpipelined: one slab of the whole problem.
  auto raggedSlab = [&]() {
    using Set0 = std::integral_constant<int, 0>;
    if constexpr (DMA) // nothing may still be on its way into buffer 0
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    loadGlobalChecked(ktBegin + nkFull, Set0{});
    __syncthreads(); // no wavefront still reads a full slab from buffer 0
    storeLds(0, Set0{});
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KSTEPS; kk++) {
      loadFrags(0, kk, fa[0], fb[0]);
      tieFragments(fa[0], fb[0], TieNow{});
#pragma unroll
      for (int m = 0; m < NM; m++)
        acc[m / NI][m % NI] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            fb[0][m % NI], fa[0][m / NI], acc[m / NI][m % NI], 0, 0, 0);
    }
    __syncthreads(); // buffer 0 may be rewritten
  };
  if constexpr (!kLatencyFirst) {
    if (hasTail)
      raggedSlab(); // buffer 0 is rewritten by the first full slab afterwards
  }
  if (nk > 0) {
    if constexpr (!kLatencyFirst)
      staticFor<DIST>(
          [&](auto d) { loadGlobal(ktBegin + decltype(d)::value, d); });
    if constexpr (DMA) {
      // slabs 0 .. DIST-1 are on their way to buffers 0 .. DIST-1; slab 0 has
      // landed when the DIST-1 slabs behind it are all that is outstanding
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((DIST - 1) * NV)
                   : "memory");
    } else {
      storeLds(0, std::integral_constant<int, 0>{});
      loadGlobal(ktBegin + DIST, std::integral_constant<int, 0>{});
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    if constexpr (kWholeSlabFrags) {
      staticFor<KSTEPS>([&](auto kkC) {
        constexpr int kk = decltype(kkC)::value;
        loadFrags(0, kk, fa[kk % FSETS], fb[kk % FSETS]);
      });
    } else {
      loadFrags(0, 0, fa[0], fb[0]);
    }
    auto oneSlab = [&](int idx, auto setC, auto tailC) {
      if constexpr (kWholeSlabFrags)
        slabWhole(idx, setC, tailC);
      else
        slab(idx, setC, tailC);
    };
    int i = 0;
    for (; i + DIST < nk; i += DIST) {
      staticFor<DIST>([&](auto d) {
        constexpr int D = decltype(d)::value;
        oneSlab(i + D, std::integral_constant<int, (D + 1) % DIST>{},
                std::false_type{});
      });
    }
    bool go = true;
    staticFor<DIST>([&](auto d) {
      constexpr int D = decltype(d)::value;
      go = go && i + D < nk;
      if (go)
        oneSlab(i + D, std::integral_constant<int, (D + 1) % DIST>{},
                std::true_type{});
    });
  }
  if constexpr (kLatencyFirst) {
    if (hasTail)
      raggedSlab(); // behind the full slabs, whose requests went out first
  }
  if constexpr (DMA) // the ring's last requests (never read) land before LDS is reused
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  static_assert(WM * WN * 32 * (WTN * 4 + 16) +
                        (EPI >= kEpiFoldA ? BM * 8 * (1 + WN) : 0) <=
                    NBUF * STAGE_BYTES,
                "epilogue strips (and the row statistics of the folded "
                "epilogues behind them) must fit the main loop's LDS");
  if constexpr (EPI >= kEpiFoldA) {
    if constexpr (!kFoldEarly)
      foldStat = foldRowStatFinish<BM>(p, m0, tid, foldRaw);
    epilogueFold<MI, NI, WTM, WTN, EPI, BM, THREADS>(p, acc, m0, n0, waveM,
                                                     waveN, lane, wave, tid,
                                                     foldStat, smem);
  } else if (numSlices > 1) {
    storePartial<MI, NI, THREADS>(p, acc, tile, slice, numSlices, tid);
    if constexpr (EPI < kEpiRowStats) {
      if (p.tileArrivals != nullptr &&
          arriveAtTile(p, tile, numSlices, tid, smem)) {
        sumPartials<MI, NI, THREADS>(p, acc, tile, numSlices, tid);
        epilogueAuto<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane,
                                            wave, smem);
      }
    }
  } else
    epilogueAuto<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane,
                                        wave, smem);
  vpid += gridDim.x;
  } while (vpid < nTiles); // tiles of this workgroup
}

template <int BM, int BN, int WM, int WN, int DIST, int EPI, bool B_NK,
          bool DMA = false>
Status launchPipe(const GemmProblem &pr, hipStream_t s) {
  constexpr int SMEM = (DMA ? DIST + 1 : 2) * (BM + BN) * 64 * 2;
  static_assert(!DMA || ((BM * 8) % (WM * WN * kWave) == 0 &&
                         (BN * 8) % (WM * WN * kWave) == 0 &&
                         (B_NK || 1024 % (BN * 2) == 0 || (BN * 2) % 1024 == 0)),
                "a DMA instruction fills 1 KiB: whole rows of the tile");
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
  auto kernel = gemmPipeKernel<BM, BN, WM, WN, DIST, EPI, B_NK, DMA>;
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
  GemmParams q = plan.p;
  // The slices of a tile are workgroups x, x + gridX, x + 2 gridX ... of the
  // launch: with gridX a multiple of the XCD count they share an XCD, and the
  // last of them to finish can sum the partial tiles itself.
  bool sumInKernel = false;
  if (plan.splitK > 1 && plan.splitK <= 64 && EPI < kEpiRowStats &&
      !plan.callerWorkspace &&
      (gridX % kNumXcd == 0 || splitKInKernelMode() == 2) &&
      (splitKInKernelMode() != 3 ||
       splitKInKernelPays(BM * BN, plan.splitK, plan.nTiles)) &&
      plan.nTiles <= kMaxArrivalTiles) {
    SplitKArrival arr;
    if (splitKArrival(s, &arr)) {
      q.tileArrivals = arr.words;
      q.misplaced = arr.misplaced;
      sumInKernel = true;
    }
  }
  // (leading dimensions fit 31 bits: checked above)
  kernel<<<dim3((unsigned)gridX, (unsigned)plan.splitK), dim3(WM * WN * kWave),
           SMEM, s>>>(q.A, q.B, q.M, q.N, q.K, int(q.lda), int(q.ldb), q.tilesN,
                      q.xcdQ,
                      uint32_t(q.xcdR) | uint32_t(q.lastRows) << 4 |
                          uint32_t(q.fullGroups) << 8,
                      q.groupMagic, q.kTilesPerSlice, q);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  if (plan.splitK > 1 && !sumInKernel)
    return launchReduce<BM, BN, WM, WN, EPI, 8>(plan, s);
  return Status::kSuccess;
}

} // namespace gemmk
} // namespace hom
