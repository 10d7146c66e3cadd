// mvllm_silu_and_mul: SiluAndMul.forward, src/myvllm/layers/activation.py:15-18
//   x, y = input.chunk(2, dim=-1);  out = silu(x) * y
// Rounding follows the two tensor operations: silu(x) = x / (1 + exp(-x)) in fp32 rounded to the element type,
// then the product in fp32 rounded again.  One launch, 16-byte accesses, rows of the GEMM output as they lie.
#include "common.h"

#pragma clang fp contract(off)

namespace mvllm {

constexpr int kActThreads = 256;

template <typename T> struct Act8 {
  static constexpr int N = 8;    // elements per 16-byte access
  static __device__ __forceinline__ void load(const T* p, float (&x)[8]) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    x[0] = lo_to_float<T>(w.x); x[1] = hi_to_float<T>(w.x);
    x[2] = lo_to_float<T>(w.y); x[3] = hi_to_float<T>(w.y);
    x[4] = lo_to_float<T>(w.z); x[5] = hi_to_float<T>(w.z);
    x[6] = lo_to_float<T>(w.w); x[7] = hi_to_float<T>(w.w);
  }
  static __device__ __forceinline__ void store(T* p, const float (&x)[8]) {
    T o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = from_float<T>(x[e]);
    *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(o);
  }
};
template <> struct Act8<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float (&x)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  }
};

template <typename T>
__global__ __launch_bounds__(kActThreads) void silu_and_mul_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                                   int64_t rows, int width, int64_t in_stride) {
  constexpr int N = Act8<T>::N;
  const int per_row = width / N;                                   // vector accesses per output row
  const int64_t total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * kActThreads + threadIdx.x; i < total; i += (int64_t)gridDim.x * kActThreads) {
    const int64_t r = i / per_row;
    const int c = (int)(i - r * per_row) * N;
    float a[8], b[8], y[8];
    Act8<T>::load(in + r * in_stride + c, a);
    Act8<T>::load(in + r * in_stride + width + c, b);
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float s = to_float(from_float<T>(a[e] / (1.0f + __expf(-a[e]))));
      y[e] = s * b[e];
    }
    Act8<T>::store(out + r * (int64_t)width + c, y);
  }
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_silu_and_mul(void* out, const void* in, int64_t rows, int width, int64_t in_row_stride, int dtype,
                                  void* stream) {
  const int esize = dtype_size(dtype);
  if (esize == 0) return MVLLM_ERR_BAD_DTYPE;
  if (rows < 0 || width <= 0 || in_row_stride < 2 * (int64_t)width) return MVLLM_ERR_BAD_SHAPE;
  const int n = 16 / esize;
  if (width % n != 0 || in_row_stride % n != 0) return MVLLM_ERR_UNSUPPORTED;
  if (rows == 0) return MVLLM_OK;
  if (!out || !in) return MVLLM_ERR_NULL_POINTER;
  if (!aligned16(out) || !aligned16(in)) return MVLLM_ERR_MISALIGNED;
  const int64_t total = rows * (width / n);
  int64_t blocks = (total + kActThreads - 1) / kActThreads;
  if (blocks > 65536) blocks = 65536;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks), block(kActThreads);
  switch (dtype) {
    case MVLLM_F32: silu_and_mul_kernel<float><<<grid, block, 0, s>>>((float*)out, (const float*)in, rows, width, in_row_stride); break;
    case MVLLM_BF16: silu_and_mul_kernel<bf16_t><<<grid, block, 0, s>>>((bf16_t*)out, (const bf16_t*)in, rows, width, in_row_stride); break;
    default: silu_and_mul_kernel<f16_t><<<grid, block, 0, s>>>((f16_t*)out, (const f16_t*)in, rows, width, in_row_stride); break;
  }
  return launch_status();
}
