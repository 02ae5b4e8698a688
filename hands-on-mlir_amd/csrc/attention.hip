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
// One wavefront owns 32 query rows; a workgroup of NW wavefronts shares the
// K / V blocks (64 keys at a time) through LDS.  Both contractions run on
// v_mfma_f32_32x32x16_f16 and are issued transposed:
//   S^T = K Q^T   (A operand = K rows, B operand = Q rows, both contiguous in d)
//   O^T = V^T P^T (A operand = V columns, B operand = P rows)
// With that orientation a lane holds, for ONE query row, 16 of the 32 scores of
// a key sub-block, so the online-softmax row reductions are in-lane plus one
// exchange with lane^32, and the probabilities are already laid out as the B
// operand of the second MFMA: P never leaves registers.  The MFMA k index is
// free as long as both operands agree, so V is read in the key order the score
// accumulators happen to have.  V is staged as (key, key+1) half2 pairs so that
// those reads are conflict-free 32-bit LDS loads.
#include "kernels.h"

namespace hom {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kHeadDim = 64;
constexpr int kKeyBlock = 64;
constexpr int K_LD = kHeadDim + 8;  // halves per LDS row of K
constexpr int VP_LD = kHeadDim + 16; // dwords per LDS row of key-pair-packed V

template <int NW>
__global__ __launch_bounds__(NW *kWave) void bertAttentionKernel(
    const _Float16 *__restrict__ qkv, const int32_t *__restrict__ cu,
    _Float16 *__restrict__ out, int seq, int heads, float scale) {
  constexpr int kThreads = NW * kWave;
  __shared__ __attribute__((aligned(16))) _Float16 sK[kKeyBlock * K_LD];
  __shared__ __attribute__((aligned(16))) uint32_t sV[(kKeyBlock / 2) * VP_LD];

  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int l32 = lane % 32, hb = lane / 32;
  const int head = blockIdx.y, b = blockIdx.z;
  const int q0 = blockIdx.x * (NW * 32) + wave * 32;
  int len = cu[b + 1] - cu[b];
  len = len < 0 ? 0 : (len > seq ? seq : len);

  const int64_t tokStride = int64_t(3) * heads * kHeadDim;
  const _Float16 *base = qkv + int64_t(b) * seq * tokStride;
  const _Float16 *qBase = base + head * kHeadDim;
  const _Float16 *kBase = base + (heads + head) * kHeadDim;
  const _Float16 *vBase = base + (2 * heads + head) * kHeadDim;
  const int64_t outStride = int64_t(heads) * kHeadDim;
  _Float16 *oBase = out + int64_t(b) * seq * outStride + head * kHeadDim;

  // A workgroup whose query rows are all padding has nothing to compute.
  if (int(blockIdx.x) * (NW * 32) >= len) {
    const int q = q0 + l32;
    if (q < seq) {
      half4 z;
#pragma unroll
      for (int e = 0; e < 4; e++)
        z[e] = _Float16(0);
#pragma unroll
      for (int c = 0; c < 8; c++)
        *reinterpret_cast<half4 *>(oBase + int64_t(q) * outStride + c * 8 +
                                   hb * 4) = z;
    }
    return;
  }

  // Q fragments (B operand of S^T = K Q^T): lane (q = l32, hb) holds
  // Q[q][kk*16 + hb*8 .. +8] for kk = 0..3.
  half8 fq[kHeadDim / 16];
  {
    const int q = q0 + l32;
#pragma unroll
    for (int kk = 0; kk < kHeadDim / 16; kk++) {
      half8 v;
#pragma unroll
      for (int e = 0; e < 8; e++)
        v[e] = _Float16(0);
      if (q < seq)
        v = *reinterpret_cast<const half8 *>(qBase + int64_t(q) * tokStride +
                                             kk * 16 + hb * 8);
      fq[kk] = v;
    }
  }

  float16v accO[2]; // O^T: two 32-wide d blocks
#pragma unroll
  for (int d = 0; d < 2; d++)
#pragma unroll
    for (int e = 0; e < 16; e++)
      accO[d][e] = 0.f;
  float rowMax = -INFINITY, rowSum = 0.f;

  // The whole workgroup walks the same key blocks (uniform trip count).
  const int numBlocks = (len + kKeyBlock - 1) / kKeyBlock;
  for (int kbIdx = 0; kbIdx < numBlocks; kbIdx++) {
    const int key0 = kbIdx * kKeyBlock;
    __syncthreads(); // previous block fully consumed
    // ---- stage K: 64 keys x 8 vectors of 16 bytes ----
    for (int v = tid; v < kKeyBlock * (kHeadDim / 8); v += kThreads) {
      const int r = v / (kHeadDim / 8), c = (v % (kHeadDim / 8)) * 8;
      half8 val;
#pragma unroll
      for (int e = 0; e < 8; e++)
        val[e] = _Float16(0);
      if (key0 + r < seq)
        val = *reinterpret_cast<const half8 *>(
            kBase + int64_t(key0 + r) * tokStride + c);
      *reinterpret_cast<half8 *>(sK + r * K_LD + c) = val;
    }
    // ---- stage V as (key, key+1) pairs ----
    for (int v = tid; v < (kKeyBlock / 2) * (kHeadDim / 8); v += kThreads) {
      const int kp = v / (kHeadDim / 8), c = (v % (kHeadDim / 8)) * 8;
      half8 v0, v1;
#pragma unroll
      for (int e = 0; e < 8; e++)
        v0[e] = v1[e] = _Float16(0);
      const int key = key0 + 2 * kp;
      if (key < seq)
        v0 = *reinterpret_cast<const half8 *>(vBase + int64_t(key) * tokStride +
                                              c);
      if (key + 1 < seq)
        v1 = *reinterpret_cast<const half8 *>(
            vBase + int64_t(key + 1) * tokStride + c);
      half8 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        lo[2 * e] = v0[e];
        lo[2 * e + 1] = v1[e];
        hi[2 * e] = v0[4 + e];
        hi[2 * e + 1] = v1[4 + e];
      }
      *reinterpret_cast<half8 *>(sV + kp * VP_LD + c) = lo;
      *reinterpret_cast<half8 *>(sV + kp * VP_LD + c + 4) = hi;
    }
    __syncthreads();

    // ---- S^T = K Q^T for two 32-key sub-blocks ----
    float16v accS[2];
#pragma unroll
    for (int sb = 0; sb < 2; sb++) {
#pragma unroll
      for (int e = 0; e < 16; e++)
        accS[sb][e] = 0.f;
#pragma unroll
      for (int kk = 0; kk < kHeadDim / 16; kk++) {
        const half8 fk = *reinterpret_cast<const half8 *>(
            sK + (sb * 32 + l32) * K_LD + kk * 16 + hb * 8);
        accS[sb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk, fq[kk], accS[sb],
                                                          0, 0, 0);
      }
    }
    // accS[sb][e] is the score of query l32 against key
    //   key0 + sb*32 + 8*(e/4) + 4*hb + e%4.
    float blockMax = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < 2; sb++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int key = key0 + sb * 32 + 8 * (e / 4) + 4 * hb + (e % 4);
        const float s = key < len ? accS[sb][e] * scale : -INFINITY;
        accS[sb][e] = s;
        blockMax = fmaxf(blockMax, s);
      }
    blockMax = fmaxf(blockMax, __shfl_xor(blockMax, 32, kWave));
    const float newMax = fmaxf(rowMax, blockMax);
    // Every block that is visited has at least one valid key, so newMax is
    // finite and the differences below are never inf - inf.
    const float corr = __expf(rowMax - newMax);
    float blockSum = 0.f;
#pragma unroll
    for (int sb = 0; sb < 2; sb++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const float pv = __expf(accS[sb][e] - newMax);
        accS[sb][e] = pv;
        blockSum += pv;
      }
    blockSum += __shfl_xor(blockSum, 32, kWave);
    rowSum = rowSum * corr + blockSum;
    rowMax = newMax;
#pragma unroll
    for (int d = 0; d < 2; d++)
#pragma unroll
      for (int e = 0; e < 16; e++)
        accO[d][e] *= corr;

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
        for (int d = 0; d < 2; d++) {
          // A operand: V[key(hb, e)][d*32 + l32]; keys come in two runs of 4 =
          // two pairs each.
          uint4v w;
#pragma unroll
          for (int g = 0; g < 2; g++) {
            const int keyLocal = sb * 32 + 8 * (2 * t + g) + 4 * hb;
            const int kp = keyLocal / 2;
            w[2 * g] = sV[kp * VP_LD + d * 32 + l32];
            w[2 * g + 1] = sV[(kp + 1) * VP_LD + d * 32 + l32];
          }
          const half8 fv = __builtin_bit_cast(half8, w);
          accO[d] =
              __builtin_amdgcn_mfma_f32_32x32x16_f16(fv, fp, accO[d], 0, 0, 0);
        }
      }
    }
  }

  // ---- normalise and store ----
  // accO[d][e]: column dcol = d*32 + 8*(e/4) + 4*hb + e%4 of query row l32.
  const int q = q0 + l32;
  if (q < seq) {
    const bool valid = q < len;
    const float inv = valid ? 1.0f / rowSum : 0.f;
#pragma unroll
    for (int d = 0; d < 2; d++)
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
  HOM_CHECK_RET(headDim == kHeadDim, Status::kInvalidArgument,
                "attention: head size %lld not supported (only 64)",
                (long long)headDim);
  HOM_CHECK_RET(bs < 65536 && heads < 65536 && seq < (int64_t(1) << 24),
                Status::kInvalidArgument, "attention: shape out of range");
  HOM_CHECK_RET((reinterpret_cast<uintptr_t>(qkv) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 7) == 0,
                Status::kInvalidArgument, "attention: misaligned operands");
  if (bs == 0 || seq == 0 || heads == 0)
    return Status::kSuccess;
  // Fewer wavefronts per workgroup when there are few (batch, head) pairs, so
  // that short sequences still spread over the chip.
  const int cus = deviceInfo().computeUnits;
  const int64_t pairs = bs * heads;
  if (pairs * ((seq + 127) / 128) >= 2 * int64_t(cus)) {
    dim3 grid((unsigned)((seq + 127) / 128), (unsigned)heads, (unsigned)bs);
    bertAttentionKernel<4><<<grid, dim3(256), 0, s>>>(qkv, cuSeqlens, out,
                                                      int(seq), int(heads),
                                                      scale);
  } else if (pairs * ((seq + 63) / 64) >= int64_t(cus)) {
    dim3 grid((unsigned)((seq + 63) / 64), (unsigned)heads, (unsigned)bs);
    bertAttentionKernel<2><<<grid, dim3(128), 0, s>>>(qkv, cuSeqlens, out,
                                                      int(seq), int(heads),
                                                      scale);
  } else {
    dim3 grid((unsigned)((seq + 31) / 32), (unsigned)heads, (unsigned)bs);
    bertAttentionKernel<1><<<grid, dim3(64), 0, s>>>(qkv, cuSeqlens, out,
                                                     int(seq), int(heads),
                                                     scale);
  }
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

} // namespace hom
