// mvllm_add_rms_norm: the decoder layer's residual add + RMSNorm in one launch.
// Reference: LayerNorm.forward / residual_rms_forward / rms_forward, src/myvllm/layers/layernorm.py:9-28
//   x = x + residual                                   (in the element type: the sum is rounded to it)
//   out = x / sqrt(mean(x^2) + eps) * gamma, residual_out = x
// as called twice per layer and once after the last layer (src/myvllm/models/qwen3.py:197-212, 306-312).
// The norm is computed in fp32 from the rounded sum with separate multiplies and adds (no contraction), a
// correctly rounded square root and the quotient x / denominator taken with one correction step from the
// correctly rounded reciprocal (SharedDivisor); only the order of the sum of squares is free.
//
// One wave per row; lane l holds elements [8 (l + 64 c), +8) for chunks c = 0 .. CHUNKS-1 in registers, so the
// row is read once and written once (16-byte accesses).
#include "common.h"

#pragma clang fp contract(off)

namespace mvllm {

template <typename T> struct Row8;
template <> struct Row8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
  }
};
template <typename T16> struct Row8 {
  static __device__ __forceinline__ void load(const T16* p, float (&x)[8]) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    x[0] = lo_to_float<T16>(w.x); x[1] = hi_to_float<T16>(w.x);
    x[2] = lo_to_float<T16>(w.y); x[3] = hi_to_float<T16>(w.y);
    x[4] = lo_to_float<T16>(w.z); x[5] = hi_to_float<T16>(w.z);
    x[6] = lo_to_float<T16>(w.w); x[7] = hi_to_float<T16>(w.w);
  }
  static __device__ __forceinline__ void store(T16* p, const float (&x)[8]) {
    T16 o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = from_float<T16>(x[e]);
    *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(o);
  }
};

constexpr int kNormThreads = 256;   // 4 rows per workgroup

template <typename T, int CHUNKS>
__global__ __launch_bounds__(kNormThreads) void add_rms_norm_kernel(
    T* __restrict__ out, T* __restrict__ residual_out, const T* __restrict__ x, const T* __restrict__ residual,
    const float* __restrict__ gamma, float eps, int64_t rows, int hidden, int64_t x_stride, int64_t res_stride) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kNormThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xp = x + row * x_stride;
  float v[CHUNKS][8];
  // gamma does not depend on the row: for short rows it is fetched together with the row instead of after the
  // reduction, which takes one memory latency out of a kernel that is all latency at decode batch sizes
  constexpr bool kEarlyGamma = CHUNKS <= 4;
  float gam[kEarlyGamma ? CHUNKS : 1][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int e0 = 8 * (lane + 64 * c);
    if (e0 < hidden) {
      Row8<T>::load(xp + e0, v[c]);
      if constexpr (kEarlyGamma) Row8<float>::load(gamma + e0, gam[c]);
      if (residual) {
        float r[8];
        Row8<T>::load(residual + row * res_stride + e0, r);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] = to_float(from_float<T>(v[c][e] + r[e]));   // the sum lives in T
      }
      if (residual_out) Row8<T>::store(residual_out + row * (int64_t)hidden + e0, v[c]);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = ss + v[c][e] * v[c][e];
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ss = ss + __shfl_xor(ss, o, 64);
  const SharedDivisor denom(sqrtf(ss / (float)hidden + eps));
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int e0 = 8 * (lane + 64 * c);
    if (e0 < hidden) {
      float g[8], y[8];
      if constexpr (kEarlyGamma) {
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] = gam[c][e];
      } else {
        Row8<float>::load(gamma + e0, g);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = denom.divide(v[c][e]) * g[e];
      Row8<T>::store(out + row * (int64_t)hidden + e0, y);
    }
  }
}

template <typename T>
static int launch_norm(void* out, void* residual_out, const void* x, const void* residual, const float* gamma, float eps,
                       int64_t rows, int hidden, int64_t x_stride, int64_t res_stride, hipStream_t s) {
  const int chunks = (hidden + 511) / 512;
  const dim3 grid((unsigned)((rows + kNormThreads / 64 - 1) / (kNormThreads / 64))), block(kNormThreads);
#define MVLLM_LAUNCH_N(C)                                                                                      \
  add_rms_norm_kernel<T, C><<<grid, block, 0, s>>>((T*)out, (T*)residual_out, (const T*)x, (const T*)residual, \
                                                   gamma, eps, rows, hidden, x_stride, res_stride)
  if (chunks <= 1) MVLLM_LAUNCH_N(1);
  else if (chunks <= 2) MVLLM_LAUNCH_N(2);
  else if (chunks <= 4) MVLLM_LAUNCH_N(4);
  else if (chunks <= 8) MVLLM_LAUNCH_N(8);
  else MVLLM_LAUNCH_N(16);
#undef MVLLM_LAUNCH_N
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_add_rms_norm(void* out, void* residual_out, const void* x, const void* residual,
                                  const float* gamma, float eps, int64_t rows, int hidden, int64_t x_row_stride,
                                  int64_t residual_row_stride, int dtype, void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (rows < 0 || hidden <= 0 || x_row_stride < hidden || (residual && residual_row_stride < hidden))
    return MVLLM_ERR_BAD_SHAPE;
  if (hidden % 8 != 0 || hidden > 8192) return MVLLM_ERR_UNSUPPORTED;
  if (rows == 0) return MVLLM_OK;
  if (!out || !x || !gamma) return MVLLM_ERR_NULL_POINTER;
  if (!aligned16(out) || !aligned16(x) || !aligned16(gamma) || (residual && !aligned16(residual)) ||
      (residual_out && !aligned16(residual_out)) || ((x_row_stride | residual_row_stride) & 7) != 0)
    return MVLLM_ERR_MISALIGNED;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MVLLM_F32:
      return launch_norm<float>(out, residual_out, x, residual, gamma, eps, rows, hidden, x_row_stride, residual_row_stride, s);
    case MVLLM_BF16:
      return launch_norm<bf16_t>(out, residual_out, x, residual, gamma, eps, rows, hidden, x_row_stride, residual_row_stride, s);
    default:
      return launch_norm<f16_t>(out, residual_out, x, residual, gamma, eps, rows, hidden, x_row_stride, residual_row_stride, s);
  }
}
