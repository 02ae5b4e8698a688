// Layer norm over the last dimension for gfx950.
//
// Semantics follow the reference's LayernormRunner (include/NVGPUKernels/
// Layernorm.h:584-694): statistics in fp32, biased variance, y = (x - mean) *
// rsqrt(var + eps); the reference form has no affine parameters and runs in
// place.  The optional residual / gamma / beta operands are a superset.
//
// The kernel is bandwidth bound: each row is read once with 128-bit loads and
// stays in registers for the two statistic passes; one 64-lane wavefront owns
// a row and reduces across lanes inside the vector ALU (no LDS).  Rows that do not fit
// that scheme (odd lengths, very long rows) take a workgroup-per-row kernel
// that reduces through LDS.
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

// One wavefront per row; VPL 16-byte vectors per lane.
//
// STREAM == false: tensors of a few megabytes, which the next kernel of the
// stream finds in the last-level cache (results written through, see
// store_policy.h).  STREAM == true: tensors beyond that cache; rows are read
// and written with the non-temporal hint, because nothing is touched twice and
// without the hint the written rows linger in the L2s and compete with the
// reads on their way out (16384 x 1024 in place, rotating over 800 MB so that
// every launch is cold: 4.5 TB/s with default accesses, 5.4 TB/s with the hint,
// 5.6 TB/s with the in-place form's stores also written through; a plain
// read-modify-write probe shows the same 4.65 -> 5.55 -> 5.72 TB/s.  With a
// residual operand, two read streams and a write stream, writing through costs
// 1 % instead: 17.4 against 17.5 us).
//
// The kernel is a chain of memory round trips (arguments, row, result) a few
// hundred nanoseconds each, so everything it will read is requested at once and
// nothing stands between the requests: a lane without a vector of its own
// (768 columns: lanes 32..63 of the second vector) and a wavefront past the
// last row load a valid address again and mask the values, instead of a branch
// around the load, which would make the second request wait for the first.
template <typename T, int VPL, bool HAS_RES, bool HAS_AFFINE, bool STREAM>
__global__ __launch_bounds__(256) void layernormWaveKernel(
    const T *x, const T *res,
    const T *__restrict__ gamma, const T *__restrict__ beta, T *out,
    int64_t rows, int hidden, float eps) {
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::kN;
  constexpr int kRowsPerBlock = 256 / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  // the same for every lane of a wavefront: row addresses stay scalar
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t rowWant = int64_t(blockIdx.x) * kRowsPerBlock + wave;
  const bool rowOk = rowWant < rows;
  const int64_t row = rowOk ? rowWant : rows - 1;
  const int nvec = hidden / N;
  const V *xr = reinterpret_cast<const V *>(x + row * hidden);
  const V *rr = HAS_RES ? reinterpret_cast<const V *>(res + row * hidden)
                        : nullptr;

  V raw[VPL];
  V rawRes[VPL];
  V g[VPL], b[VPL];
  const bool hasG = HAS_AFFINE && gamma != nullptr;
  const bool hasB = HAS_AFFINE && beta != nullptr;
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int idx = lane + i * kWave;
    const int at = idx < nvec ? idx : 0;
    raw[i] = STREAM ? __builtin_nontemporal_load(&xr[at]) : xr[at];
    if (HAS_RES)
      rawRes[i] = STREAM ? __builtin_nontemporal_load(&rr[at]) : rr[at];
    if (HAS_AFFINE) {
      // (null gamma / beta: wave-uniform branches, taken by nobody or everybody)
      if (hasG)
        g[i] = reinterpret_cast<const V *>(gamma)[at];
      if (hasB)
        b[i] = reinterpret_cast<const V *>(beta)[at];
    }
  }
  // every request is out before the first value is touched
  __builtin_amdgcn_sched_barrier(0);
  float v[VPL][N];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const bool mine = lane + i * kWave < nvec;
#pragma unroll
    for (int j = 0; j < N; j++) {
      float f = float(raw[i][j]);
      if (HAS_RES)
        f += float(rawRes[i][j]); // the sum stays in fp32
      f = mine ? f : 0.f;
      v[i][j] = f;
      sum += f;
    }
  }
  const float invH = 1.0f / float(hidden);
  const float mean = waveSum(sum) * invH;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const bool mine = lane + i * kWave < nvec;
#pragma unroll
    for (int j = 0; j < N; j++) {
      const float d = mine ? v[i][j] - mean : 0.f;
      sq += d * d;
    }
  }
  const float var = waveSum(sq) * invH;
  const float rstd = 1.0f / sqrtf(var + eps);

  V *orow = reinterpret_cast<V *>(out + row * hidden);
#pragma unroll
  for (int i = 0; i < VPL; i++) {
    const int idx = lane + i * kWave;
    V o;
#pragma unroll
    for (int j = 0; j < N; j++) {
      float y = (v[i][j] - mean) * rstd;
      if (hasG)
        y *= float(g[i][j]);
      if (hasB)
        y += float(b[i][j]);
      o[j] = T(y);
    }
    if (rowOk && idx < nvec) {
      if (STREAM && !HAS_RES)
        storeStreaming(&orow[idx], o); // the in-place form: see store_policy.h
      else if (STREAM)
        __builtin_nontemporal_store(o, &orow[idx]);
      else
        storeWriteThrough(&orow[idx], o);
    }
  }
}

__device__ __forceinline__ float blockSum(float v, float *lds) {
  v = waveSum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = blockDim.x / kWave;
  __syncthreads(); // lds may still be read from a previous reduction
  if (lane == 0)
    lds[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; i++)
    total += lds[i];
  return total;
}

// One workgroup per row, any row length, scalar accesses.
template <typename T>
__global__ __launch_bounds__(256) void layernormBlockKernel(
    const T *x, const T *res,
    const T *__restrict__ gamma, const T *__restrict__ beta, T *out,
    int64_t rows, int64_t hidden, float eps) {
  __shared__ float lds[8];
  const int64_t row = blockIdx.x;
  const T *xr = x + row * hidden;
  const T *rr = res ? res + row * hidden : nullptr;
  T *orow = out + row * hidden;
  auto load = [&](int64_t i) -> float {
    float f = float(xr[i]);
    if (rr)
      f += float(rr[i]);
    return f;
  };
  float sum = 0.f;
  for (int64_t i = threadIdx.x; i < hidden; i += blockDim.x)
    sum += load(i);
  const float mean = blockSum(sum, lds) / float(hidden);
  float sq = 0.f;
  for (int64_t i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float d = load(i) - mean;
    sq += d * d;
  }
  const float var = blockSum(sq, lds) / float(hidden);
  const float rstd = 1.0f / sqrtf(var + eps);
  // All reads of this row are done (blockSum synchronised) before any write,
  // so out may alias x.
  for (int64_t i = threadIdx.x; i < hidden; i += blockDim.x) {
    float y = (load(i) - mean) * rstd;
    if (gamma)
      y *= float(gamma[i]);
    if (beta)
      y += float(beta[i]);
    orow[i] = T(y);
  }
}

// Results that the next kernel of the stream will find in the last-level cache
// (a few megabytes) are written through; larger tensors stream.
constexpr int64_t kSmallTensorBytes = int64_t(16) << 20;

#define HOM_LN_LAUNCH(KERNEL, ...)                                             \
  do {                                                                         \
    if (res) {                                                                 \
      if (affine)                                                              \
        KERNEL<T, VPL, true, true, ##__VA_ARGS__>                              \
            <<<grid, block, 0, s>>>(x, res, gamma, beta, out, rows, hidden, eps); \
      else                                                                     \
        KERNEL<T, VPL, true, false, ##__VA_ARGS__>                             \
            <<<grid, block, 0, s>>>(x, res, gamma, beta, out, rows, hidden, eps); \
    } else {                                                                   \
      if (affine)                                                              \
        KERNEL<T, VPL, false, true, ##__VA_ARGS__>                             \
            <<<grid, block, 0, s>>>(x, res, gamma, beta, out, rows, hidden, eps); \
      else                                                                     \
        KERNEL<T, VPL, false, false, ##__VA_ARGS__>                            \
            <<<grid, block, 0, s>>>(x, res, gamma, beta, out, rows, hidden, eps); \
    }                                                                          \
  } while (0)

template <typename T, int VPL>
void launchWave(const T *x, const T *res, const T *gamma, const T *beta, T *out,
                int64_t rows, int hidden, float eps, hipStream_t s) {
  const int rowsPerBlock = 256 / kWave;
  dim3 grid((unsigned)((rows + rowsPerBlock - 1) / rowsPerBlock)), block(256);
  const bool affine = gamma || beta;
  if (rows * hidden * int64_t(sizeof(T)) <= kSmallTensorBytes) {
    HOM_LN_LAUNCH(layernormWaveKernel, false);
  } else {
    // (a persistent variant whose wavefronts keep their next row in flight
    // while they reduce and store the current one measured the same 12.3-12.6
    // us on 16384 x 1024 cold, at 2 to 8 workgroups per CU: the rate is the
    // memory system's for a read-modify-write stream of this size)
    HOM_LN_LAUNCH(layernormWaveKernel, true);
  }
}
#undef HOM_LN_LAUNCH

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

} // namespace

template <typename T>
Status launchLayernorm(const T *x, const T *res, const T *gamma, const T *beta,
                       T *out, int64_t rows, int64_t hidden, float eps,
                       hipStream_t s) {
  if (rows == 0 || hidden == 0)
    return Status::kSuccess;
  HOM_CHECK_RET(rows < (int64_t(1) << 31), Status::kInvalidArgument,
                "layernorm: too many rows (%lld)", (long long)rows);
  constexpr int N = Vec16<T>::kN;
  const bool vecOk = hidden % N == 0 && aligned16(x) && aligned16(out) &&
                     (!res || aligned16(res)) && (!gamma || aligned16(gamma)) &&
                     (!beta || aligned16(beta));
  const int64_t nvec = hidden / N;
  if (vecOk && nvec <= kWave * 8) {
    const int h = int(hidden);
    if (nvec <= kWave)
      launchWave<T, 1>(x, res, gamma, beta, out, rows, h, eps, s);
    else if (nvec <= kWave * 2)
      launchWave<T, 2>(x, res, gamma, beta, out, rows, h, eps, s);
    else if (nvec <= kWave * 4)
      launchWave<T, 4>(x, res, gamma, beta, out, rows, h, eps, s);
    else
      launchWave<T, 8>(x, res, gamma, beta, out, rows, h, eps, s);
  } else {
    layernormBlockKernel<T><<<dim3((unsigned)rows), dim3(256), 0, s>>>(
        x, res, gamma, beta, out, rows, hidden, eps);
  }
  HOM_HIP_RET(hipGetLastError(), Status::kInternal);
  return Status::kSuccess;
}

template Status launchLayernorm<_Float16>(const _Float16 *, const _Float16 *,
                                          const _Float16 *, const _Float16 *,
                                          _Float16 *, int64_t, int64_t, float,
                                          hipStream_t);
template Status launchLayernorm<float>(const float *, const float *,
                                       const float *, const float *, float *,
                                       int64_t, int64_t, float, hipStream_t);

} // namespace hom
