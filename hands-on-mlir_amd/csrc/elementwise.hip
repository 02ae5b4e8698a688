// Bandwidth-bound helper kernels for gfx950: broadcasting binary elementwise
// ops, embedding gather, cu_seqlens, GELU, and the row-statistic kernels of the
// LN-GEMM pair.  All use 128-bit accesses where shape and alignment allow.
//
// Reference semantics:
//   elementwise  include/NVGPUKernels/ElementwiseRunner.h:69-153
//   gather       include/NVGPUKernels/GatherRunner.h:32-77
//   cu_seqlens   include/NVGPUKernels/CuSeqLen.h:28-74
//   row stats    include/NVGPUKernels/Layernorm.h:33-195 (ApplyFinalReduction)
#include "cross_lane.h"
#include "kernels.h"
#include "store_policy.h"

namespace hom {
namespace {

constexpr int kWave = 64;

template <typename T> struct Vec16;
template <> struct Vec16<_Float16> {
  static constexpr int kN = 8;
  typedef _Float16 type __attribute__((ext_vector_type(8)));
};
template <> struct Vec16<float> {
  static constexpr int kN = 4;
  typedef float type __attribute__((ext_vector_type(4)));
};

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

template <typename T> __device__ __forceinline__ T applyOp(int op, T a, T b) {
  switch (op) {
  case 0:
    return a + b;
  case 1:
    return a - b;
  case 2:
    return a * b;
  default:
    // fp16 division goes through fp32 (correctly rounded there, then rounded
    // to fp16), like a half division on the reference's hardware.
    return T(float(a) / float(b));
  }
}

// Out = A op B with B either the same shape (inner == total) or repeating
// every `inner` elements (broadcast over leading dimensions).  One 16-byte
// vector per thread per step.
template <typename T, int OP>
__global__ __launch_bounds__(256) void elementwiseVecKernel(
    const T *a, const T *b, T *out, int64_t nvec, int64_t innerVec) {
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::kN;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec;
       i += step) {
    const V va = reinterpret_cast<const V *>(a)[i];
    const V vb = reinterpret_cast<const V *>(b)[i % innerVec];
    V vo;
#pragma unroll
    for (int j = 0; j < N; j++)
      vo[j] = applyOp<T>(OP, va[j], vb[j]);
    reinterpret_cast<V *>(out)[i] = vo;
  }
}

// Same-shape operands beyond the last-level cache: one vector per thread, every
// access with the non-temporal hint (nothing is touched twice; measured cold on
// 16384 x 1024 fp16 triples rotating over 800 MB: 5.2 TB/s with default
// accesses and a grid-stride loop, 5.9 TB/s this way).
template <typename T, int OP>
__global__ __launch_bounds__(256) void elementwiseStreamKernel(
    const T *a, const T *b, T *out, int64_t nvec) {
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::kN;
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= nvec)
    return;
  const V va = __builtin_nontemporal_load(reinterpret_cast<const V *>(a) + i);
  const V vb = __builtin_nontemporal_load(reinterpret_cast<const V *>(b) + i);
  V vo;
#pragma unroll
  for (int j = 0; j < N; j++)
    vo[j] = applyOp<T>(OP, va[j], vb[j]);
  __builtin_nontemporal_store(vo, reinterpret_cast<V *>(out) + i);
}

// Any broadcast pattern, scalar accesses.  The index walk is the reference's:
// coordinate = x / stride, clamped to B's extent, times B's stride.
template <typename T, int OP>
__global__ __launch_bounds__(256) void elementwiseGenericKernel(
    const T *a, const T *b, T *out, int64_t total, BroadcastDesc d) {
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += step) {
    int64_t x = i, bIdx = 0;
    for (int k = 0; k < d.rank; k++) {
      const int64_t coord = x / d.outStride[k];
      x -= coord * d.outStride[k];
      bIdx += (coord < d.bSize[k] ? coord : d.bSize[k] - 1) * d.bStride[k];
    }
    out[i] = applyOp<T>(OP, a[i], b[bIdx]);
  }
}

// Operands larger than this are not expected to be found in the last-level
// cache by whoever reads the result next.
constexpr int64_t kStreamingBytes = int64_t(16) << 20;

template <typename T, int OP>
Status elementwiseDispatch(const T *a, const T *b, T *out, int64_t total,
                           const BroadcastDesc &d, hipStream_t s) {
  constexpr int N = Vec16<T>::kN;
  // inner = number of trailing elements over which B is dense and contiguous;
  // every dimension in front of them must have B extent 1.
  int64_t inner = 1;
  int k = d.rank - 1;
  for (; k >= 0; k--) {
    if (d.bSize[k] != d.outSize[k] ||
        (d.outSize[k] != 1 && d.bStride[k] != inner))
      break;
    inner *= d.outSize[k];
  }
  bool leadingOnly = true;
  for (int j = k; j >= 0; j--)
    leadingOnly = leadingOnly && d.bSize[j] == 1;
  const int cus = deviceInfo().computeUnits;
  if (leadingOnly && inner % N == 0 && total % N == 0 && aligned16(a) &&
      aligned16(b) && aligned16(out)) {
    const int64_t nvec = total / N;
    int64_t blocks = (nvec + 255) / 256;
    if (inner == total && total * int64_t(sizeof(T)) > kStreamingBytes &&
        blocks < (int64_t(1) << 31)) {
      elementwiseStreamKernel<T, OP>
          <<<dim3((unsigned)blocks), dim3(256), 0, s>>>(a, b, out, nvec);
      HOM_HIP_RET(hipGetLastError(), Status::kInternal);
      return Status::kSuccess;
    }
    if (blocks > int64_t(cus) * 16)
      blocks = int64_t(cus) * 16;
    elementwiseVecKernel<T, OP><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(
        a, b, out, nvec, inner / N);
  } else {
    int64_t blocks = (total + 255) / 256;
    if (blocks > int64_t(cus) * 32)
      blocks = int64_t(cus) * 32;
    elementwiseGenericKernel<T, OP>
        <<<dim3((unsigned)blocks), dim3(256), 0, s>>>(a, b, out, total, d);
  }
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

// ---------------------------------------------------------------- gather --
template <typename T>
__global__ __launch_bounds__(256) void gatherVecKernel(
    const int64_t *__restrict__ indices, const T *__restrict__ value,
    T *__restrict__ out, int64_t numIndices, int64_t vocab, int rowVec) {
  using V = typename Vec16<T>::type;
  const int64_t total = numIndices * rowVec;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += step) {
    const int64_t r = i / rowVec;
    const int c = int(i - r * rowVec);
    int64_t src = indices[r];
    // An index outside the table would read foreign memory; clamp it.
    src = src < 0 ? 0 : (src >= vocab ? vocab - 1 : src);
    reinterpret_cast<V *>(out)[i] =
        reinterpret_cast<const V *>(value)[src * rowVec + c];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gatherScalarKernel(
    const int64_t *__restrict__ indices, const T *__restrict__ value,
    T *__restrict__ out, int64_t numIndices, int64_t vocab, int64_t rowLength) {
  const int64_t total = numIndices * rowLength;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += step) {
    const int64_t r = i / rowLength;
    const int64_t c = i - r * rowLength;
    int64_t src = indices[r];
    src = src < 0 ? 0 : (src >= vocab ? vocab - 1 : src);
    out[i] = value[src * rowLength + c];
  }
}

// ------------------------------------------------------------ cu_seqlens --
// One workgroup: each wavefront sums rows of the mask, then thread 0 runs the
// (short) inclusive scan.  Row sums pass through the output buffer itself.
template <typename InT>
__global__ __launch_bounds__(256) void cuSeqLenKernel(
    const InT *__restrict__ mask, int32_t *out, int64_t bs, int64_t seq) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = blockDim.x / kWave;
  for (int64_t r = wave; r < bs; r += nwaves) {
    int32_t sum = 0;
    for (int64_t j = lane; j < seq; j += kWave)
      sum += int32_t(mask[r * seq + j]);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1)
      sum += __shfl_xor(sum, off, kWave);
    if (lane == 0)
      out[r + 1] = sum;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t acc = 0;
    out[0] = 0;
    for (int64_t r = 0; r < bs; r++) {
      acc += out[r + 1];
      out[r + 1] = acc;
    }
  }
}

// ------------------------------------------------------------------ gelu --
__device__ __forceinline__ float geluErf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float geluTanh(float x) {
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(u));
}

template <int FORM>
__global__ __launch_bounds__(256) void geluKernel(const _Float16 *in,
                                                  _Float16 *out,
                                                  int64_t total) {
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += step) {
    const float x = float(in[i]);
    out[i] = _Float16(FORM == 0 ? geluErf(x) : geluTanh(x));
  }
}

// ------------------------------------------------------------- row stats --
__global__ __launch_bounds__(256) void rowStatsKernel(
    const _Float16 *__restrict__ d, _Float16 *__restrict__ var,
    _Float16 *__restrict__ mean, int64_t rows, int64_t n, float eps) {
  const int lane = threadIdx.x % kWave;
  const int64_t row =
      int64_t(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (row >= rows)
    return;
  float s = 0.f, sq = 0.f;
  for (int64_t j = lane; j < n; j += kWave) {
    const float x = float(d[row * n + j]);
    s += x;
    sq += x * x;
  }
  s = waveSum(s);
  sq = waveSum(sq);
  if (lane == 0) {
    const float m = s / float(n);
    const float ms = sq / float(n);
    // E[x^2] - E[x]^2 cancels to a small negative number for near-constant
    // rows; clamped so that a tiny eps cannot turn it into a NaN
    const float rstd = 1.0f / sqrtf(fmaxf(ms - m * m, 0.f) + eps);
    var[row] = _Float16(rstd);
    mean[row] = _Float16(-m * rstd);
  }
}

__global__ __launch_bounds__(256) void applyRowStatsKernel(
    const _Float16 *__restrict__ a, const _Float16 *__restrict__ var,
    const _Float16 *__restrict__ mean, _Float16 *__restrict__ out,
    int64_t rows, int64_t k) {
  const int64_t total = rows * k;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += step) {
    const int64_t r = i / k;
    out[i] = _Float16(float(a[i]) * float(var[r]) + float(mean[r]));
  }
}

inline unsigned cappedBlocks(int64_t work, int perBlock, int mult) {
  int64_t blocks = (work + perBlock - 1) / perBlock;
  const int64_t cap = int64_t(deviceInfo().computeUnits) * mult;
  if (blocks > cap)
    blocks = cap;
  if (blocks < 1)
    blocks = 1;
  return (unsigned)blocks;
}

} // namespace

template <typename T>
Status launchElementwise(BinOp op, const T *a, const T *b, T *out,
                         int64_t total, const BroadcastDesc &desc,
                         hipStream_t s) {
  if (total == 0)
    return Status::kSuccess;
  switch (op) {
  case BinOp::kAdd:
    return elementwiseDispatch<T, 0>(a, b, out, total, desc, s);
  case BinOp::kSub:
    return elementwiseDispatch<T, 1>(a, b, out, total, desc, s);
  case BinOp::kMul:
    return elementwiseDispatch<T, 2>(a, b, out, total, desc, s);
  case BinOp::kDiv:
    return elementwiseDispatch<T, 3>(a, b, out, total, desc, s);
  }
  return Status::kInvalidArgument;
}
template Status launchElementwise<_Float16>(BinOp, const _Float16 *,
                                            const _Float16 *, _Float16 *,
                                            int64_t, const BroadcastDesc &,
                                            hipStream_t);
template Status launchElementwise<float>(BinOp, const float *, const float *,
                                         float *, int64_t,
                                         const BroadcastDesc &, hipStream_t);

template <typename T>
Status launchGather(const int64_t *indices, const T *value, T *out,
                    int64_t numIndices, int64_t vocab, int64_t rowLength,
                    hipStream_t s) {
  if (numIndices == 0 || rowLength == 0)
    return Status::kSuccess;
  constexpr int N = Vec16<T>::kN;
  if (rowLength % N == 0 && aligned16(value) && aligned16(out) &&
      rowLength / N < (int64_t(1) << 31)) {
    const int rowVec = int(rowLength / N);
    gatherVecKernel<T>
        <<<dim3(cappedBlocks(numIndices * rowVec, 256, 16)), dim3(256), 0, s>>>(
            indices, value, out, numIndices, vocab, rowVec);
  } else {
    gatherScalarKernel<T>
        <<<dim3(cappedBlocks(numIndices * rowLength, 256, 32)), dim3(256), 0,
           s>>>(indices, value, out, numIndices, vocab, rowLength);
  }
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}
template Status launchGather<_Float16>(const int64_t *, const _Float16 *,
                                       _Float16 *, int64_t, int64_t, int64_t,
                                       hipStream_t);
template Status launchGather<float>(const int64_t *, const float *, float *,
                                    int64_t, int64_t, int64_t, hipStream_t);

template <typename InT>
Status launchCuSeqLen(const InT *mask, int32_t *out, int64_t bs, int64_t seq,
                      hipStream_t s) {
  cuSeqLenKernel<InT><<<dim3(1), dim3(256), 0, s>>>(mask, out, bs, seq);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}
template Status launchCuSeqLen<int64_t>(const int64_t *, int32_t *, int64_t,
                                        int64_t, hipStream_t);
template Status launchCuSeqLen<int32_t>(const int32_t *, int32_t *, int64_t,
                                        int64_t, hipStream_t);

Status launchGeluF16(const _Float16 *in, _Float16 *out, int64_t total, int form,
                     hipStream_t s) {
  if (total == 0)
    return Status::kSuccess;
  const dim3 grid(cappedBlocks(total, 256, 32)), block(256);
  if (form == 0)
    geluKernel<0><<<grid, block, 0, s>>>(in, out, total);
  else
    geluKernel<1><<<grid, block, 0, s>>>(in, out, total);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

Status launchRowStatsF16(const _Float16 *d, _Float16 *var, _Float16 *mean,
                         int64_t rows, int64_t n, float eps, hipStream_t s) {
  if (rows == 0)
    return Status::kSuccess;
  rowStatsKernel<<<dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s>>>(
      d, var, mean, rows, n, eps);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

Status launchApplyRowStatsF16(const _Float16 *a, const _Float16 *var,
                              const _Float16 *mean, _Float16 *out, int64_t rows,
                              int64_t k, hipStream_t s) {
  if (rows == 0 || k == 0)
    return Status::kSuccess;
  applyRowStatsKernel<<<dim3(cappedBlocks(rows * k, 256, 32)), dim3(256), 0,
                        s>>>(a, var, mean, out, rows, k);
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

} // namespace hom
