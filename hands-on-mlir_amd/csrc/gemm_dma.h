// "dma" main loop: K is walked in 64-wide slabs through an NS-deep ring of LDS
// buffers filled by buffer_load_dwordx4 ... lds, i.e. global memory -> LDS
// without passing through registers.  The loads of slab k+NS-1 are in flight
// while slab k is multiplied.  Out-of-range rows/columns/k are given an offset
// beyond the buffer descriptor's size, for which the hardware writes zeros.
// LDS rows are not padded (the DMA writes 1 KiB contiguous per wavefront); bank
// conflicts are avoided by permuting 16-byte chunks inside a row, which costs
// nothing because every lane chooses its own global address.  A (and B when it
// is [N, K]) fragments are 128-bit LDS reads.  Row-major B has N contiguous
// while an MFMA operand wants 8 consecutive k per lane: those fragments are read
// with ds_read_b64_tr_b16, which transposes 4 k-rows x 16 columns across a group
// of 16 lanes.
#pragma once

#include "gemm_device.h"

namespace hom {
namespace gemmk {

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

  int tileM, tileN;
  const int tile = tileCoordsFast(p, int(blockIdx.x), &tileM, &tileN);
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
  // A slab's loads are one constant 32-bit offset per lane plus a scalar
  // offset per slab: the main loop computes no addresses and tests no ranges.
  // Rows past M (or N, for B as [N, K]) lie beyond the descriptor and read as
  // zero; columns of a row-major B past N get an offset beyond every
  // descriptor; rows of a row-major B past K lie beyond its descriptor.  Only
  // the partial last slab of a ragged K needs a test per lane (issueChecked).
  const int kEnd = ktEnd * BK < p.K ? ktEnd * BK : p.K;
  const int ktPartial = kEnd % BK != 0 ? ktEnd - 1 : -1;
  uint32_t aOff[A_PER_W];
  int aCol[A_PER_W];
#pragma unroll
  for (int i = 0; i < A_PER_W; i++) {
    const int instr = wave * A_PER_W + i;
    const int r = instr * 8 + lane / 8;
    const int c = swzK(r, lane % 8); // logical chunk stored at this position
    aCol[i] = c * 8;
    aOff[i] = (uint32_t(r) * uint32_t(p.lda) + uint32_t(c * 8)) * 2u;
  }
  uint32_t bOff[B_PER_W];
  int bK[B_PER_W]; // NK: column offset in k (KN: unused)
#pragma unroll
  for (int i = 0; i < B_PER_W; i++) {
    const int instr = wave * B_PER_W + i;
    if (B_NK) {
      const int r = instr * 8 + lane / 8;
      const int c = swzK(r, lane % 8);
      bK[i] = c * 8;
      bOff[i] = (uint32_t(r) * uint32_t(p.ldb) + uint32_t(c * 8)) * 2u;
    } else {
      constexpr int CHUNKS = B_ROW_BYTES / 16;
      const int k = instr * B_ROWS_PER_INSTR + lane / CHUNKS;
      const int pc = lane % CHUNKS; // physical chunk
      const int g = swzN<BN>(k, pc / 4);
      const int n = (g * 4 + pc % 4) * 8;
      bK[i] = 0;
      bOff[i] = (n0 + n < p.N)
                    ? (uint32_t(k) * uint32_t(p.ldb) + uint32_t(n0 + n)) * 2u
                    : kOob;
    }
  }

  auto issue = [&](int kt, int stage) {
    unsigned char *sA = smem + stage * STAGE_BYTES;
    unsigned char *sB = sA + A_BYTES;
    const int k0 = kt * BK;
    const uint32_t sOffA = uint32_t(k0) * 2u;
    const uint32_t sOffB = B_NK ? sOffA : uint32_t(k0) * uint32_t(p.ldb) * 2u;
    if (kt != ktPartial) {
#pragma unroll
      for (int i = 0; i < A_PER_W; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrcA, HOM_LDS_PTR(sA + (wave * A_PER_W + i) * 1024), 16, aOff[i],
            sOffA, 0, 0);
#pragma unroll
      for (int i = 0; i < B_PER_W; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrcB, HOM_LDS_PTR(sB + (wave * B_PER_W + i) * 1024), 16, bOff[i],
            sOffB, 0, 0);
    } else {
      // the partial slab: vectors at or past the end of K read as zero
#pragma unroll
      for (int i = 0; i < A_PER_W; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrcA, HOM_LDS_PTR(sA + (wave * A_PER_W + i) * 1024), 16,
            k0 + aCol[i] < kEnd ? aOff[i] : kOob, sOffA, 0, 0);
#pragma unroll
      for (int i = 0; i < B_PER_W; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rsrcB, HOM_LDS_PTR(sB + (wave * B_PER_W + i) * 1024), 16,
            (!B_NK || k0 + bK[i] < kEnd) ? bOff[i] : kOob, sOffB, 0, 0);
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
  // A wavefront issues LOADS_PER_TILE DMA loads per slab, in slab order, so
  // "slab j has landed for this wavefront" is vmcnt <= LOADS_PER_TILE x (slabs
  // issued after j); the barrier behind that wait makes it true for the whole
  // workgroup.  Slabs that do not exist are not issued, and the wait counts
  // what was.  Inside a slab the fragments of k step kk+1 are fetched from LDS
  // before the MFMAs of step kk are issued (two register sets), and the barrier
  // that frees the slab's LDS buffer sits between the last fragment fetch and
  // the last MFMA group, so the matrix core keeps running while the wavefronts
  // synchronise, refill the ring and fetch the next slab's first fragments.
  // The waits and the barrier are opaque asm statements with a memory clobber:
  // the compiler may not move LDS reads or DMA issues across them.
  constexpr int KSTEPS = BK / 16;
  auto waitOutstanding = [&](int slabs) { // wave-uniform, 0 .. NS-2
    staticFor<NS - 1>([&](auto vC) {
      constexpr int v = decltype(vC)::value;
      if (slabs == v)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(v * LOADS_PER_TILE) : "memory");
    });
  };
  half8 fa[2][MI], fb[2][NI];
  const int nk = ktEnd - ktBegin;
  if (nk > 0) {
    int issued = 0;
#pragma unroll
    for (int s0 = 0; s0 < NS - 1; s0++)
      if (s0 < nk) {
        issue(ktBegin + s0, s0);
        issued = s0 + 1;
      }
    waitOutstanding(issued - 1); // slab 0
    asm volatile("s_barrier" ::: "memory");
    if (issued < nk) {
      issue(ktBegin + issued, issued % NS);
      issued++;
    }
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
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        waitOutstanding(issued - i - 2);
        asm volatile("s_barrier" ::: "memory");
        if (issued < nk) {
          issue(ktBegin + issued, cur); // slab i + NS takes the buffer of slab i
          issued++;
        }
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
  epilogueAuto<MI, NI, WTM, WTN, EPI>(p, acc, m0, n0, waveM, waveN, lane, wave,
                                      smem);
#endif
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

} // namespace gemmk
} // namespace hom
