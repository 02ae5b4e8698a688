// Packed-QKV BERT self-attention with a key-padding mask, for gfx950.
//
//   QKV [bs, seq, 3, heads, 64] fp16 (per token: Q of all heads, then K, then V
//   -- the packing produced by the weight concatenation in
//   lib/Dialect/HOM/HOMFusionPass.cpp:317-346, TransformerEngine layout BS3HD),
//   cu_seqlens int32 [bs+1], Out [bs, seq, heads, 64].
//   Per (b, h):  S = scale * Q K^T over keys < len_b;  P = softmax(S) in fp32;
//   O = P V.  Query rows >= len_b are written as zeros.
// Replaces the cuDNN fused attention reached through
// include/NVGPUKernels/BertAttentionRunner.h:113-136.
//
// A workgroup of four wavefronts handles 128 or 64 query rows of one (batch,
// head): each wavefront owns 32 rows and walks every key block (long
// sequences, many workgroups), or two wavefronts share 32 rows and take every
// other key block (short sequences: fewer workgroups than CUs, the key walk of
// one wavefront is the critical path; the two halves are merged through LDS).
// Keys are walked in chunks of 128: the whole workgroup stages the chunk's K
// and V rows into LDS (one barrier), then the wavefronts run over it in blocks
// of 64 keys without further synchronisation.
// Both contractions run on v_mfma_f32_32x32x16_f16 and are issued transposed:
//   S^T = K Q^T   (A operand = K rows from LDS, B operand = Q rows in registers)
//   O^T = V^T P^T (A operand = V columns, B operand = P rows)
// With that orientation a lane holds, for ONE query row, 16 of the 32 scores of
// a key sub-block, so the online-softmax row reductions are in-lane plus one
// exchange with lane^32, and the probabilities already have the layout of the
// second MFMA's B operand: P never leaves registers.  The MFMA k index is free
// as long as both operands agree, so V is read in the key order the score
// accumulators happen to have: two runs of 4 consecutive keys per lane, each one
// ds_read_b64_tr_b16 (the transposing LDS read) from the row-major V tile.
// LDS rows are 128 bytes, unpadded; 16-byte chunks (K) / 64-byte groups (V) are
// XOR-permuted by row so that the fragment reads are bank-conflict free.
#include "cross_lane.h"
#include "kernels.h"

#include <cstring>

namespace hom {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;
// Head sizes 64, 128, 192 and 256 (template parameter D; the reference's
// contract is head size % 64 == 0).  64 is what every BERT configuration has
// and what the kernel is tuned for, 128 is the same code with twice the
// registers, 192 and 256 are functional (one wavefront per SIMD, half the keys
// per LDS chunk, staging addresses computed per vector).  A K or V row in LDS
// is D halves: 128 bytes = 8 chunks of 16 bytes = 2 groups of 64 bytes for
// D = 64.
//
// Keys staged per barrier: 128, or 64 where two tiles of 128 rows would not fit
// the 64 KB of static LDS.
template <int D> struct Chunk {
  static constexpr int value = D <= 128 ? 128 : 64;
};
// chunk c (16 bytes) of K row r lives at position c ^ ((r >> 1) & 7) (rows of
// 128 bytes: two consecutive rows cover all banks once) or c ^ (r & 15) (rows
// of 256 or 512 bytes: every row starts at bank 0), so that the 128-bit
// fragment reads of 16 consecutive rows hit 16 distinct bank groups; rows of
// 384 bytes (24 chunks) permute inside groups of 8 chunks so that a position
// never leaves the row
template <int D> __device__ __forceinline__ int swzK(int row, int chunk) {
  return D == 64    ? chunk ^ ((row >> 1) & 7)
         : D == 192 ? chunk ^ (row & 7)
                    : chunk ^ (row & 15);
}
// 64-byte group g of V row k lives at position g ^ ((k >> 1) & 1), or
// g ^ (k & 3) for rows whose group count is a multiple of 4: a transposing read
// touches 64 bytes of each of rows k..k+3
template <int D> __device__ __forceinline__ int swzV(int k, int group) {
  return D == 64 || D == 192 ? group ^ ((k >> 1) & 1) : group ^ (k & 3);
}

// NW wavefronts per workgroup, KS of them share each group of 32 query rows
// and split its key blocks between them (KS = 1: every wavefront walks all
// keys of its own 32 rows; KS = 2: half the serial work per wavefront, for
// short sequences where there are fewer workgroups than CUs and the key walk
// of one wavefront is the critical path; the halves are merged through LDS).
template <int NW, int KS, int D>
__global__ __launch_bounds__(NW *kWave)
__attribute__((amdgpu_waves_per_eu(D == 64 ? 2 : 1, D == 64 && KS == 1 ? 4 : (D <= 128 ? 2 : 1)))) void bertAttentionKernel(
    const _Float16 *__restrict__ qkv, const int32_t *__restrict__ cu,
    _Float16 *__restrict__ out, int seq, int heads, int numQTiles, int pairs,
    float scale) {
  static_assert(D == 64 || D == 128 || D == 192 || D == 256, "head size");
  static_assert(D <= 128 || KS == 1, "the key-split variant stages 128 keys per chunk");
  constexpr int kChunk = Chunk<D>::value;
  constexpr int kHeadDim = D;
  constexpr int kRowB = D * 2;               // bytes of a K or V row
  constexpr int CPR = D / 8;                 // 16-byte chunks per row
  constexpr int kTileBytes = kChunk * kRowB; // one K or V chunk in LDS
  constexpr int kThreads = NW * kWave;
  constexpr int QG = NW / KS; // groups of 32 query rows per workgroup
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * kTileBytes];
  unsigned char *const sK = smem, *const sV = smem + kTileBytes;

  const int tid = threadIdx.x, lane = tid % kWave;
  // (the same for every lane: what depends on it stays in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int l32 = lane % 32, hb = lane / 32;
  const int qg = wave % QG, kh = wave / QG; // query group, key share
  // Workgroup id -> (query tile, head, batch).  Workgroups are dealt to the 8
  // XCDs round-robin by id, and the query tiles of one (batch, head) read the
  // same K and V: ids that differ by 8 (same XCD, launched back to back) walk
  // the query tiles of one pair, so K/V are fetched into one L2 once instead
  // of once per XCD.  Needs the pair count to be a multiple of 8; the
  // 2-wavefront variant (few workgroups, launch-bound) keeps the plain order.
  // The key-split variant is launched on a (query tile, head, batch) grid: the
  // same order of workgroups as a flat id, without the divisions that would
  // stand between the kernel's entry and its first loads.
  int qTile, head, b;
  if (KS == 1) {
    const int id = blockIdx.x;
    int pair;
    if (pairs % 8 == 0) {
      const int t = id / 8;
      qTile = t % numQTiles;
      pair = (t / numQTiles) * 8 + id % 8;
    } else {
      qTile = id % numQTiles;
      pair = id / numQTiles;
    }
    head = pair % heads;
    b = pair / heads;
  } else {
    qTile = blockIdx.x;
    head = blockIdx.y;
    b = blockIdx.z;
  }
  const int q0 = qTile * (QG * 32) + qg * 32;
  const int cuLo = cu[b], cuHi = cu[b + 1]; // consumed after the first loads are out
  __builtin_amdgcn_sched_barrier(0); // requested here, not where they are consumed

  const int64_t tokStride = int64_t(3) * heads * kHeadDim;
  const _Float16 *base = qkv + int64_t(b) * seq * tokStride;
  const _Float16 *qBase = base + head * kHeadDim;
  const _Float16 *kBase = base + (heads + head) * kHeadDim;
  const _Float16 *vBase = base + (2 * heads + head) * kHeadDim;
  const int64_t outStride = int64_t(heads) * kHeadDim;
  _Float16 *oBase = out + int64_t(b) * seq * outStride + head * kHeadDim;

  // Key-split variant (short sequences, few workgroups: latency is what
  // counts): K and V rows of a 128-key chunk travel global -> registers -> LDS,
  // 16 bytes per vector.  The loads are unconditional (rows past the end of the tensor
  // are clamped, rows past the sequence end are zeroed on the way to LDS), so
  // the first chunk's loads and the Q loads are issued before the sequence
  // length has arrived.  The other variant serves long sequences with many
  // workgroups per CU, which cover each other's staging; there the early loads
  // are wasted on all-padding workgroups, and prefetching the next chunk into
  // registers measured 3-8 % slower than loading each chunk when it is due
  // (also with barriers that do not wait for the prefetch).
  // (D = 128: the prefetched rows would take 64 more registers than there are)
  constexpr bool kPrefetch = KS == 2 && D == 64;
  constexpr int VPT = kChunk * CPR / kThreads; // vectors of K (and of V) per thread
  half8 rk[VPT], rv[VPT];
  auto loadChunk = [&](int key0) {
#pragma unroll
    for (int i = 0; i < VPT; i++) {
      const int v = tid + i * kThreads;
      const int r = v / CPR, c = v % CPR;
      const int row = key0 + r < seq ? key0 + r : seq - 1;
      rk[i] = *reinterpret_cast<const half8 *>(kBase + int64_t(row) * tokStride + c * 8);
      rv[i] = *reinterpret_cast<const half8 *>(vBase + int64_t(row) * tokStride + c * 8);
    }
  };
  if (kPrefetch)
    loadChunk(0);
  // Q fragments (B operand of S^T = K Q^T): lane (q = l32, hb) holds
  // Q[q][kk*16 + hb*8 .. +8] for kk = 0..3, pre-multiplied by nothing: the scale
  // is applied to the fp32 scores.
  half8 fq[kHeadDim / 16];
  {
    // rows past the tensor are clamped: what they produce is never stored
    const int q = q0 + l32 < seq ? q0 + l32 : seq - 1;
#pragma unroll
    for (int kk = 0; kk < kHeadDim / 16; kk++)
      fq[kk] = *reinterpret_cast<const half8 *>(qBase + int64_t(q) * tokStride +
                                                kk * 16 + hb * 8);
  }

  int len = cuHi - cuLo;
  len = len < 0 ? 0 : (len > seq ? seq : len);
  // A workgroup whose query rows are all padding has nothing to compute.  (Not
  // in the key-split variant: an early exit ahead of the first use of the
  // prefetched rows lets the compiler move their loads behind the test, i.e.
  // behind the arrival of the sequence length.  Such a workgroup walks one
  // empty chunk there and stores zeros at the end.)
  if (KS == 1 && qTile * (QG * 32) >= len) {
    const int q = q0 + l32;
    if (q < seq && kh == 0) {
      half4 z;
#pragma unroll
      for (int e = 0; e < 4; e++)
        z[e] = _Float16(0);
#pragma unroll
      for (int c = 0; c < CPR; c++)
        *reinterpret_cast<half4 *>(oBase + int64_t(q) * outStride + c * 8 +
                                   hb * 4) = z;
    }
    return;
  }

  constexpr int DB = D / 32;
  float16v accO[DB]; // O^T: 32-wide d blocks
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int e = 0; e < 16; e++)
      accO[d][e] = 0.f;
  // rowMax: reference of the exponent, in raw (unscaled) score units
  float rowMax = -INFINITY, rowSum = 0.f;
  const float scaleLog2e = scale * 1.44269504088896340736f;

  // Per-lane constants of the fragment addresses.
  const int swzLane = swzK<D>(l32, 0);         // K: the row term for row = 32*x + l32
  const int trRow = (lane % 16) / 4;           // V: source row inside a run of 4 keys
  const int trCol = ((lane % 32) / 16) * 16 + (lane % 4) * 4;
  const int vSwz = swzV<D>(trRow, 0);          // key bases are multiples of 4

  // Staging without prefetch: thread t copies 16-byte vector t % 8 of rows
  // t / 8 + i * kThreads / 8.  Both swizzles depend on row bits that the
  // per-vector row step (a multiple of 16) leaves alone, so the LDS
  // destinations are one base plus immediates.
  // (Head sizes above 128: the row step is not a multiple of 16, or not a
  // whole number; those compute every vector's addresses, see below.)
  constexpr bool kFastStage = kThreads % CPR == 0 && (kThreads / CPR) % 16 == 0;
  static_assert(kFastStage || D > 128, "row step per vector must leave the swizzles alone");
  const uint32_t rowBytes = uint32_t(tokStride) * 2u;
  const uint32_t stageOff = uint32_t(tid / CPR) * rowBytes + uint32_t(tid % CPR) * 16u;
  const int stageK = (tid / CPR) * kRowB + swzK<D>(tid / CPR, tid % CPR) * 16;
  const int stageV = (tid / CPR) * kRowB + swzV<D>(tid / CPR, (tid % CPR) / 4) * 64 +
                     ((tid % CPR) % 4) * 16;
  const auto rsrcK = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(kBase), 0, int32_t(uint32_t(len) * rowBytes),
      0x00020000);
  const auto rsrcV = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(vBase), 0, int32_t(uint32_t(len) * rowBytes),
      0x00020000);

  // uniform over the workgroup; at least one round in the key-split variant,
  // whose first chunk is already on its way
  const int numChunks =
      KS == 2 && len <= kChunk ? 1 : (len + kChunk - 1) / kChunk;
  // (at least one round in either variant: a loop that may run zero times
  // would put a test of the sequence length ahead of the prefetched loads)
  int ch = 0;
  do {
    const int key0 = ch * kChunk;
    // keys of this chunk that any wavefront will touch, rounded up to a block
    const int live = (len - key0 < kChunk ? ((len - key0 + 63) / 64) * 64 : kChunk);
    if (ch > 0)
      __syncthreads(); // previous chunk fully consumed
    // ---- stage K and V rows [key0, key0 + live): 8 vectors of 16 bytes per row.
    // Rows past the sequence end are zero-filled: masked scores ignore K, but a
    // masked probability (0) times a non-finite V would poison the output.
    if (kPrefetch) {
#pragma unroll
      for (int i = 0; i < VPT; i++) {
        const int v = tid + i * kThreads;
        const int r = v / CPR, c = v % CPR;
        if (r < live) {
          half8 kv = rk[i], vv = rv[i];
          if (key0 + r >= len) {
#pragma unroll
            for (int e = 0; e < 8; e++)
              kv[e] = vv[e] = _Float16(0);
          }
          *reinterpret_cast<half8 *>(sK + r * kRowB + swzK<D>(r, c) * 16) = kv;
          *reinterpret_cast<half8 *>(sV + r * kRowB + swzV<D>(r, c / 4) * 64 + (c % 4) * 16) = vv;
        }
      }
    } else {
      // Whole chunk, no range tests: the descriptors end at row `len`, so rows
      // past the sequence read as zero without touching memory.  All loads go
      // out before the first LDS store; addresses are one add per vector.
      half8 kv[VPT], vv[VPT];
      if constexpr (kFastStage) {
        const uint32_t chunkOff = stageOff + uint32_t(key0) * rowBytes;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
          const uint32_t off = chunkOff + uint32_t(i * (kThreads / CPR)) * rowBytes;
          kv[i] = __builtin_bit_cast(
              half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcK, off, 0, 0));
          vv[i] = __builtin_bit_cast(
              half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcV, off, 0, 0));
        }
#pragma unroll
        for (int i = 0; i < VPT; i++) {
          *reinterpret_cast<half8 *>(sK + stageK + i * (kThreads / CPR) * kRowB) = kv[i];
          *reinterpret_cast<half8 *>(sV + stageV + i * (kThreads / CPR) * kRowB) = vv[i];
        }
      } else {
        // vector v of the chunk = 16-byte chunk v % CPR of row v / CPR
        static_assert((kChunk * CPR) % kThreads == 0, "whole vectors per thread");
#pragma unroll
        for (int i = 0; i < VPT; i++) {
          const int v = tid + i * kThreads;
          const uint32_t off =
              uint32_t(key0 + v / CPR) * rowBytes + uint32_t(v % CPR) * 16u;
          kv[i] = __builtin_bit_cast(
              half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcK, off, 0, 0));
          vv[i] = __builtin_bit_cast(
              half8, __builtin_amdgcn_raw_buffer_load_b128(rsrcV, off, 0, 0));
        }
#pragma unroll
        for (int i = 0; i < VPT; i++) {
          const int v = tid + i * kThreads;
          const int r = v / CPR, c = v % CPR;
          *reinterpret_cast<half8 *>(sK + r * kRowB + swzK<D>(r, c) * 16) = kv[i];
          *reinterpret_cast<half8 *>(sV + r * kRowB + swzV<D>(r, c / 4) * 64 +
                                     (c % 4) * 16) = vv[i];
        }
      }
    }
    if (kPrefetch && ch + 1 < numChunks)
      loadChunk(key0 + kChunk);
    __syncthreads();

    for (int blk = kh * 64; blk < live; blk += 64 * KS) {
      // ---- S^T = K Q^T for two 32-key sub-blocks ----
      // All eight K fragments are requested before the first MFMA: read one
      // at a time, each MFMA would wait out a full LDS round trip.
      // accS[sb][e] is the raw score (before scaling) of query l32 against key
      //   key0 + blk + sb*32 + 8*(e/4) + 4*hb + e%4.
      // Only a block that reaches past the sequence end pays for the key mask.
      float16v accS[2];
      auto scores = [&]() {
        half8 fk[2][kHeadDim / 16];
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
          for (int kk = 0; kk < kHeadDim / 16; kk++)
            fk[sb][kk] = *reinterpret_cast<const half8 *>(
                sK + (blk + sb * 32 + l32) * kRowB + ((kk * 2 + hb) ^ swzLane) * 16);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int sb = 0; sb < 2; sb++) {
#pragma unroll
          for (int e = 0; e < 16; e++)
            accS[sb][e] = 0.f;
#pragma unroll
          for (int kk = 0; kk < kHeadDim / 16; kk++)
            accS[sb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[sb][kk], fq[kk],
                                                              accS[sb], 0, 0, 0);
        }
        if (key0 + blk + 64 > len) {
#pragma unroll
          for (int sb = 0; sb < 2; sb++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
              const int key = key0 + blk + sb * 32 + 8 * (e / 4) + 4 * hb + (e % 4);
              accS[sb][e] = key < len ? accS[sb][e] : -INFINITY;
            }
        }
      };
      scores();
      // The softmax works on raw scores: with c = scale * log2(e) > 0,
      // exp(scale * (s - m)) = exp2(c * s - c * m), one FMA and one v_exp per
      // score; the reference m (rowMax, raw units) only has to keep p within
      // range, it need not be the true maximum, and the final O / rowSum cancels
      // whatever reference was used.  This part is VALU work the matrix core
      // cannot hide (16 MFMAs against a few hundred vector instructions per
      // block), so instruction count matters:
      //  - fast path (every block but a wavefront's first): p is computed
      //    against the reference as it stands, no maximum is taken at all, and
      //    the row sums that are needed anyway tell whether that was safe: if
      //    some row's sum over the 64 keys exceeds kSumLimit (so a p could leave
      //    fp16's range; an overflowed exp2 gives inf and lands here too) the
      //    block's scores are recomputed from LDS and take the slow path;
      //  - slow path (the first block, and a block whose sums overflowed): the
      //    true block maximum, the reference moves to it, O and the running
      //    sum are rescaled (96 vector instructions on the accumulators).
      // With real score distributions the slow path runs once per wavefront.
      // Every block that is visited has at least one valid key, so blockMax
      // is finite and the differences below are never inf - inf.
      constexpr float kSumLimit = 4096.0f;
      const bool first = ch == 0 && blk == kh * 64;
      float blockSum = 0.f;
      bool slow = first;
      if (!first) {
        const float negMax = -rowMax * scaleLog2e;
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
          for (int e = 0; e < 16; e++) {
            const float pv =
                __builtin_amdgcn_exp2f(fmaf(accS[sb][e], scaleLog2e, negMax));
            accS[sb][e] = pv;
            blockSum += pv;
          }
        blockSum = pairSum(blockSum);
        slow = __any(!(blockSum <= kSumLimit));
        if (slow)
          scores(); // the probabilities are discarded: raw scores again
      }
      if (slow) {
        float blockMax = -INFINITY;
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
          for (int e = 0; e < 16; e++)
            blockMax = fmaxf(blockMax, accS[sb][e]);
        blockMax = pairMax(blockMax);
        const float newMax = fmaxf(rowMax, blockMax);
        // (first block: rowMax = -inf, corr = 0 on accumulators that are 0)
        const float corr = __builtin_amdgcn_exp2f((rowMax - newMax) * scaleLog2e);
        rowSum *= corr;
        rowMax = newMax;
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
          for (int e = 0; e < 16; e++)
            accO[d][e] *= corr;
        const float negMax = -rowMax * scaleLog2e;
        blockSum = 0.f;
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
          for (int e = 0; e < 16; e++) {
            const float pv =
                __builtin_amdgcn_exp2f(fmaf(accS[sb][e], scaleLog2e, negMax));
            accS[sb][e] = pv;
            blockSum += pv;
          }
        blockSum = pairSum(blockSum);
      }
      rowSum += blockSum;

      // ---- O^T += V^T P^T ----
#pragma unroll
      for (int sb = 0; sb < 2; sb++) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
          // B operand: P[q][key(hb, e)], key(hb, e) = sb*32 + 8*(2t + e/4) + 4*hb
          // + e%4, which is accumulators 8t .. 8t+7 of this lane.
          half8 fp;
#pragma unroll
          for (int e = 0; e < 8; e++)
            fp[e] = _Float16(accS[sb][8 * t + e]);
#pragma unroll
          for (int d = 0; d < DB; d++) {
            // A operand: V[key(hb, e)][d*32 + l32]: two runs of 4 consecutive
            // keys, each transposed out of 4 V rows x 16 columns by one read.
            short4v run[2];
#pragma unroll
            for (int g = 0; g < 2; g++) {
              const int keyLocal = blk + sb * 32 + 8 * (2 * t + g) + 4 * hb + trRow;
              run[g] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                  (__attribute__((address_space(3))) short4v *)(
                      sV + keyLocal * kRowB + (d ^ vSwz) * 64 + trCol * 2));
            }
            short8v both;
#pragma unroll
            for (int e = 0; e < 4; e++) {
              both[e] = run[0][e];
              both[4 + e] = run[1][e];
            }
            accO[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(half8, both), fp, accO[d], 0, 0, 0);
          }
        }
      }
    }
  } while (++ch < numChunks);

  // ---- merge the key shares ----
  // Share 1 hands (reference, sum, O) of its rows to share 0 through LDS, in
  // the layout [query group][value][lane]; lanes of the two wavefronts hold
  // the same (row, columns).  With references m0, m1 in raw score units and
  // m = max(m0, m1): O = O0 2^((m0-m)c) + O1 2^((m1-m)c), the same for the
  // sums.  A share that saw no valid key has m1 = -inf and weight 0; share 0
  // always owns the first block, which has one.
  if constexpr (KS == 2) {
    constexpr int XV = DB * 16; // accumulator values per lane
    static_assert(QG * (XV + 2) * kWave * 4 <= 2 * kTileBytes, "exchange fits the K/V tiles");
    float *xch = reinterpret_cast<float *>(smem) + qg * ((XV + 2) * kWave) + lane;
    __syncthreads(); // every wavefront is done with K and V
    if (kh == 1) {
#pragma unroll
      for (int d = 0; d < DB; d++)
#pragma unroll
        for (int e = 0; e < 16; e++)
          xch[(d * 16 + e) * kWave] = accO[d][e];
      xch[XV * kWave] = rowMax;
      xch[(XV + 1) * kWave] = rowSum;
    }
    __syncthreads();
    if (kh == 1)
      return;
    const float m1 = xch[XV * kWave], l1 = xch[(XV + 1) * kWave];
    const float m = fmaxf(rowMax, m1);
    const float c0 = __builtin_amdgcn_exp2f((rowMax - m) * scaleLog2e);
    const float c1 = __builtin_amdgcn_exp2f((m1 - m) * scaleLog2e);
    rowSum = rowSum * c0 + l1 * c1;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        accO[d][e] = accO[d][e] * c0 + xch[(d * 16 + e) * kWave] * c1;
  }

  // ---- normalise and store ----
  // accO[d][e]: column dcol = d*32 + 8*(e/4) + 4*hb + e%4 of query row l32.
  const int q = q0 + l32;
  if (q < seq) {
    const bool valid = q < len;
    const float inv = valid ? 1.0f / rowSum : 0.f;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        half4 o;
#pragma unroll
        for (int e = 0; e < 4; e++)
          o[e] = valid ? _Float16(accO[d][g * 4 + e] * inv) : _Float16(0);
        *reinterpret_cast<half4 *>(oBase + int64_t(q) * outStride + d * 32 +
                                   g * 8 + hb * 4) = o;
      }
  }
}

} // namespace

Status launchBertAttentionF16(const _Float16 *qkv, const int32_t *cuSeqlens,
                              _Float16 *out, int64_t bs, int64_t seq,
                              int64_t heads, int64_t headDim, float scale,
                              hipStream_t s) {
  // (the reference's contract is head size % 64 == 0, README.md:11; the
  // sizes with kernels here are 64, 128, 192 and 256)
  HOM_CHECK_RET(headDim == 64 || headDim == 128 || headDim == 192 || headDim == 256,
                Status::kInvalidArgument,
                "attention: head size %lld not supported (64, 128, 192 or 256)",
                (long long)headDim);
  // The softmax tracks the maximum of the unscaled scores, which is the
  // maximum of the scaled ones only for a positive scale (BERT: 1/sqrt(64)).
  HOM_CHECK_RET(scale > 0.f, Status::kInvalidArgument,
                "attention: scale must be positive (got %g)", double(scale));
  HOM_CHECK_RET(bs < 65536 && heads < 65536 && seq < (int64_t(1) << 24),
                Status::kInvalidArgument, "attention: shape out of range");
  // K/V staging addresses a batch entry with 32-bit byte offsets
  HOM_CHECK_RET(seq * 3 * heads * headDim * 2 < (int64_t(1) << 31),
                Status::kInvalidArgument,
                "attention: one batch entry of QKV must be smaller than 2 GiB");
  HOM_CHECK_RET((reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 7) == 0,
                Status::kInvalidArgument, "attention: misaligned operands");
  if (bs == 0 || seq == 0 || heads == 0)
    return Status::kSuccess;
  // 128 query rows per workgroup (one wavefront per 32 rows) when that still
  // gives every CU work, otherwise 64 with the keys split over two wavefronts
  // per 32 rows (K/V of a (batch, head) are then staged by two workgroups).
  const int cus = deviceInfo().computeUnits;
  const int64_t pairs = bs * heads;
  bool wide = pairs * ((seq + 127) / 128) >= int64_t(cus) || seq <= 32;
  // profiling knob: HOM_ATTENTION_VARIANT=wide | split
  if (const char *force = getenv("HOM_ATTENTION_VARIANT"))
    wide = strcmp(force, "wide") == 0;
  if (headDim > 128)
    wide = true; // (the key-split variant exists for 64 and 128 only)
  HOM_CHECK_RET(pairs * ((seq + 63) / 64) < (int64_t(1) << 31),
                Status::kInvalidArgument, "attention: too many workgroups");
  if (wide) {
    const int nq = int((seq + 127) / 128);
    const dim3 grid((unsigned)(nq * pairs));
    if (headDim == 64)
      bertAttentionKernel<4, 1, 64><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
    else if (headDim == 128)
      bertAttentionKernel<4, 1, 128><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
    else if (headDim == 192)
      bertAttentionKernel<4, 1, 192><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
    else
      bertAttentionKernel<4, 1, 256><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
  } else {
    const int nq = int((seq + 63) / 64);
    HOM_CHECK_RET(heads < 65536 && bs < 65536, Status::kInvalidArgument,
                  "attention: heads and batch size must be below 65536");
    const dim3 grid((unsigned)nq, (unsigned)heads, (unsigned)bs);
    if (headDim == 64)
      bertAttentionKernel<4, 2, 64><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
    else
      bertAttentionKernel<4, 2, 128><<<grid, dim3(256), 0, s>>>(
          qkv, cuSeqlens, out, int(seq), int(heads), nq, int(pairs), scale);
  }
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

} // namespace hom
