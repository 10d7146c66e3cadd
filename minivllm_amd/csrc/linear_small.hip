// Linear layer for the few rows of a decode step: out[M, N] = x[M, K] W[N, K]^T + bias, M <= 64, bf16 / fp16.
// The caller's projections around the attention path (src/myvllm/models/qwen3.py:90-94, 118 and the MLP, :121-160;
// layers/linear.py) are library GEMMs in the reference.  With a handful of rows such a product reads a few MB of
// weights once, from HBM (a model's layers do not fit the caches together), and is pure latency: a tiled GEMM walks
// K in a serial loop of small loads.  Here a workgroup owns 16 output columns, its W waves split K, and a wave asks
// for its whole share of the weights (and of x, which stays in L2) in one or a few bursts before the first MFMA, so
// a call costs about one memory round trip.
//   per wave and 32-wide k step: A = W (row n0 + lane%16, 16 B = 8 k values of class lane/16), B = x^T (column m =
//   lane%16, the same k values), v_mfma_f32_16x16x32: lane l ends with out[m = l%16][n0 + 4 (l/16) + r], r < 4.
//   The partial sums meet in LDS; wave 0 adds them, adds the bias and stores 8 bytes per lane.
#include "common.h"

namespace mvllm {

struct LinearArgs {
  void* out;
  const void* x;
  const void* w;
  const void* bias;       // [N] in the element type, or null
  int64_t x_row_stride;   // elements between rows of x
  int M, N, K;
};

template <typename T, int MT, int U, int W>
__global__ __launch_bounds__(64 * W) void linear_small_kernel(const LinearArgs a) {
  __shared__ float4 part[(W - 1) * MT * 64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15, cls = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int ksl = a.K / W;                               // this wave's share of K
  const T* wp = reinterpret_cast<const T*>(a.w) + (int64_t)(n0 + col) * a.K + wave * ksl + cls * 8;
  const T* xp[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = min(16 * mt + col, a.M - 1);           // rows past M repeat the last one; they are not stored
    xp[mt] = reinterpret_cast<const T*>(a.x) + (int64_t)m * a.x_row_stride + wave * ksl + cls * 8;
  }
  v4f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < ksl; k += 32 * U) {
    uint4 wf[U], xf[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) wf[u] = load16_stream(wp + k + 32 * u);      // weights are read once: stream them
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int u = 0; u < U; ++u) xf[mt][u] = *reinterpret_cast<const uint4*>(xp[mt] + k + 32 * u);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = mfma16x16x32<T>(wf[u], xf[mt][u], acc[mt]);
  }
  if (wave > 0) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      part[((wave - 1) * MT + mt) * 64 + lane] = make_float4(acc[mt][0], acc[mt][1], acc[mt][2], acc[mt][3]);
  }
  __syncthreads();
  if (wave > 0) return;
  float b4[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.bias) {
    const T* bp = reinterpret_cast<const T*>(a.bias) + n0 + 4 * cls;
#pragma unroll
    for (int r = 0; r < 4; ++r) b4[r] = to_float(bp[r]);
  }
  T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float s[4] = {acc[mt][0], acc[mt][1], acc[mt][2], acc[mt][3]};
    for (int w = 0; w < W - 1; ++w) {
      const float4 p = part[(w * MT + mt) * 64 + lane];
      s[0] += p.x; s[1] += p.y; s[2] += p.z; s[3] += p.w;
    }
    const int m = 16 * mt + col;
    if (m < a.M) {
      T r4[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) r4[r] = from_float<T>(s[r] + b4[r]);
      *reinterpret_cast<uint2*>(out + (int64_t)m * a.N + n0 + 4 * cls) = *reinterpret_cast<const uint2*>(r4);
    }
  }
}

template <typename T, int W>
static int launch_linear_w(const LinearArgs& a, hipStream_t stream) {
  const dim3 grid((unsigned)(a.N / 16)), block(64 * W);
  const int mt = (a.M + 15) / 16;
  const int steps = a.K / W / 32;                        // 32-wide k steps per wave
  // loads in flight per burst: 8 steps of W and x for up to 32 rows, 4 for more (registers)
  if (mt <= 2 && steps % 8 == 0) {
    if (mt == 1) linear_small_kernel<T, 1, 8, W><<<grid, block, 0, stream>>>(a);
    else linear_small_kernel<T, 2, 8, W><<<grid, block, 0, stream>>>(a);
  } else if (steps % 4 == 0) {
    if (mt == 1) linear_small_kernel<T, 1, 4, W><<<grid, block, 0, stream>>>(a);
    else if (mt == 2) linear_small_kernel<T, 2, 4, W><<<grid, block, 0, stream>>>(a);
    else if (mt == 3) linear_small_kernel<T, 3, 4, W><<<grid, block, 0, stream>>>(a);
    else linear_small_kernel<T, 4, 4, W><<<grid, block, 0, stream>>>(a);
  } else {
    return MVLLM_ERR_UNSUPPORTED;
  }
  return launch_status();
}

// waves per workgroup: more of them share a column tile's K when N alone gives too few workgroups to keep the
// memory system busy (N = 1024: 64 column tiles)
static int linear_waves(int N, int K) {
  int w = 4;
  while (w < 16 && (int64_t)(N / 16) * w < 1024 && K % (2 * w * 128) == 0) w *= 2;
  return w;
}

template <typename T>
static int launch_linear_small(const LinearArgs& a, hipStream_t stream) {
  switch (linear_waves(a.N, a.K)) {
    case 4: return launch_linear_w<T, 4>(a, stream);
    case 8: return launch_linear_w<T, 8>(a, stream);
    default: return launch_linear_w<T, 16>(a, stream);
  }
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_linear_small_m(void* out, const void* x, const void* w, const void* bias, int64_t x_row_stride,
                                    int M, int N, int K, int dtype, void* stream) {
  if (dtype != MVLLM_BF16 && dtype != MVLLM_F16) return dtype_size(dtype) == 0 ? MVLLM_ERR_BAD_DTYPE : MVLLM_ERR_UNSUPPORTED;
  if (M < 0 || N <= 0 || K <= 0 || x_row_stride < K) return MVLLM_ERR_BAD_SHAPE;
  if (M == 0) return MVLLM_OK;
  if (!out || !x || !w) return MVLLM_ERR_NULL_POINTER;
  if (M > 64 || N % 16 != 0 || K % 512 != 0 || x_row_stride % 8 != 0) return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(w) || (reinterpret_cast<uintptr_t>(out) & 7u) || (reinterpret_cast<uintptr_t>(bias) & 7u))
    return MVLLM_ERR_MISALIGNED;
  LinearArgs a;
  a.out = out; a.x = x; a.w = w; a.bias = bias; a.x_row_stride = x_row_stride; a.M = M; a.N = N; a.K = K;
  return dtype == MVLLM_BF16 ? launch_linear_small<bf16_t>(a, (hipStream_t)stream)
                             : launch_linear_small<f16_t>(a, (hipStream_t)stream);
}
