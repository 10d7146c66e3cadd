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
// From 17 rows on every 16 rows get workgroups of their own (the same code; the workgroups of one column tile run on
// one XCD and share the weights in its L2) rather than one workgroup holding up to four row tiles in registers.
// mvllm_norm_linear_small_m is the same product with the launches around it folded in: the residual add + RMSNorm in
// front of the layer's first projections (src/myvllm/models/qwen3.py:197-212 through layers/layernorm.py:9-28) as
// the kernel's prologue, and SiluAndMul behind the gate/up projection (layers/activation.py:15-18) as its epilogue,
// each rounding where the separate launch rounds.
#include "common.h"

#pragma clang fp contract(off)

namespace mvllm {

struct LinearArgs {
  void* out;
  const void* x;
  const void* w;
  const void* bias;       // [N] in the element type, or null
  int64_t x_row_stride;   // elements between rows of x
  int M, N, K;
  int cols;               // output columns per workgroup: 16, or 8 / 4 (plain product only) to spread few columns over more CUs
  int row_tiles;          // > 1: the grid holds this many workgroups per column tile, one per 16 rows of x (MT == 1)
  // NORM: x is first replaced by rms_norm(x + residual) * gamma, as mvllm_add_rms_norm computes it
  const void* residual;   // [M, K] contiguous, or null (then the norm of x alone)
  void* residual_out;     // [M, K] contiguous: x + residual in the element type; must not alias x or residual
  const float* gamma;     // [K]
  float eps;
};

// silu(g) * u with the roundings of the two tensor operations (activation.hip): silu in fp32 rounded to T, then the
// product rounded to T
template <typename T>
__device__ __forceinline__ T silu_mul_rounded(T g, T u) {
  const float a = to_float(g);
  const float s = to_float(from_float<T>(a / (1.0f + __expf(-a))));
  return from_float<T>(s * to_float(u));
}

template <typename T>
__device__ __forceinline__ void unpack8(uint4 w, float (&x)[8]) {
  x[0] = lo_to_float<T>(w.x); x[1] = hi_to_float<T>(w.x);
  x[2] = lo_to_float<T>(w.y); x[3] = hi_to_float<T>(w.y);
  x[4] = lo_to_float<T>(w.z); x[5] = hi_to_float<T>(w.z);
  x[6] = lo_to_float<T>(w.w); x[7] = hi_to_float<T>(w.w);
}
typedef __attribute__((ext_vector_type(2))) float v2f;
typedef __attribute__((ext_vector_type(2))) __bf16 v2bf16;
typedef __attribute__((ext_vector_type(2))) _Float16 v2f16;
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){a, b}, v2bf16));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f){a, b}, v2f16));
}
template <typename T>
__device__ __forceinline__ uint4 pack8(const float (&x)[8]) {
  return make_uint4(pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3]), pack2<T>(x[4], x[5]), pack2<T>(x[6], x[7]));
}

// NORM (the wave's whole share of K is one burst, K / W == 32 U): the rows are normalised on their way into the
// product.  Every workgroup needs every row, so each of them forms h = x + residual for all rows, the waves add
// their shares of the sums of squares through LDS, and the rounded h / sqrt(mean h^2 + eps) * gamma is the B operand:
// the value the separate norm launch would have written, without the launch.  Workgroup b < M also writes row b of h
// (the next residual).
// GLU (N = 2 F, out is [M, F]): a workgroup owns 8 gate columns and the 8 up columns that meet them, and wave 0
// finishes with out = silu(gate) * up instead of storing both halves for one more launch to read back.
template <typename T, int MT, int U, int W, bool NORM, bool GLU>
__global__ __launch_bounds__(64 * W) void linear_small_kernel(const LinearArgs a) {
  __shared__ float4 part[(W - 1) * MT * 64];
  __shared__ float sumsq[NORM ? W * MT * 16 : 1];
  __shared__ __align__(16) float gam[NORM ? W * 32 * U : 4];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15, cls = lane >> 4;
  const int ksl = a.K / W;                               // this wave's share of K
  const int koff = wave * ksl + cls * 8;                 // first k of this lane in every 32-wide step
  // column tile and first row of this workgroup.  With row tiles the workgroups of one column tile read the same
  // weights: consecutive workgroups go to the eight XCDs in turn, so the row tiles of a column tile are dealt 8
  // apart and meet in one L2.
  int ct = blockIdx.x, m0 = 0;
  if (MT == 1 && a.row_tiles > 1) {
    const int tiles = gridDim.x / a.row_tiles;
    if ((tiles & 7) == 0) {
      const int g = ct >> 3;
      m0 = 16 * (g % a.row_tiles);
      ct = (g / a.row_tiles) * 8 + (ct & 7);
    } else {
      m0 = 16 * (ct % a.row_tiles);
      ct = ct / a.row_tiles;
    }
  }
  const int mrows = min(a.M - m0, 16 * MT);              // rows of this workgroup
  int wrow, n0;                                          // weight row of this lane; first output column of the workgroup
  if constexpr (GLU) {
    n0 = ct * 8;
    wrow = col < 8 ? n0 + col : a.N / 2 + n0 + col - 8;
  } else {
    n0 = ct * a.cols;
    wrow = n0 + min(col, a.cols - 1);
  }
  const bool wlive = GLU || col < a.cols;                // weight rows of a narrow tile: the other lanes load nothing
  const T* wp = reinterpret_cast<const T*>(a.w) + (int64_t)wrow * a.K + koff;
  int rowm[MT];
  const T* xp[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    rowm[mt] = m0 + min(16 * mt + col, mrows - 1);       // rows past the last repeat it; they are not stored
    xp[mt] = reinterpret_cast<const T*>(a.x) + (int64_t)rowm[mt] * a.x_row_stride + koff;
  }
  v4f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < ksl; k += 32 * U) {
    uint4 wf[U], xf[MT][U];
    if (MT == 1 && a.row_tiles > 1) {                    // the other row tiles' workgroups read the same weights: keep them in L2
#pragma unroll
      for (int u = 0; u < U; ++u)
        wf[u] = wlive ? *reinterpret_cast<const uint4*>(wp + k + 32 * u) : make_uint4(0u, 0u, 0u, 0u);
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u)                        // weights are read once: stream them
        wf[u] = wlive ? load16_stream(wp + k + 32 * u) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int u = 0; u < U; ++u) xf[mt][u] = *reinterpret_cast<const uint4*>(xp[mt] + k + 32 * u);
    if constexpr (NORM) {
      // gamma does not depend on the data: the wave's share of it is asked for with the rows (one coalesced load)
      // and waits in LDS until the sums of squares are known
      float4 gl = make_float4(0.f, 0.f, 0.f, 0.f);
      if (4 * lane < 32 * U) gl = *reinterpret_cast<const float4*>(a.gamma + wave * ksl + 4 * lane);
      float ss[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        ss[mt] = 0.f;
        const T* rp = a.residual ? reinterpret_cast<const T*>(a.residual) + (int64_t)rowm[mt] * a.K + koff : nullptr;
        uint4 rf[U];
        if (rp) {
#pragma unroll
          for (int u = 0; u < U; ++u) rf[u] = *reinterpret_cast<const uint4*>(rp + 32 * u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float h[8];
          unpack8<T>(xf[mt][u], h);
          if (rp) {
            float r[8];
            unpack8<T>(rf[u], r);
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = to_float(from_float<T>(h[e] + r[e]));   // the sum lives in T
            xf[mt][u] = pack8<T>(h);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) ss[mt] = ss[mt] + h[e] * h[e];
        }
        // the next residual: row b of the workgroup's rows is written by the workgroup of column tile b (all of
        // them hold these rows)
        if (a.residual_out && 16 * mt + col == ct && ct < mrows) {
          T* hp = reinterpret_cast<T*>(a.residual_out) + (int64_t)(m0 + ct) * a.K + koff;
#pragma unroll
          for (int u = 0; u < U; ++u) *reinterpret_cast<uint4*>(hp + 32 * u) = xf[mt][u];
        }
        ss[mt] = ss[mt] + __shfl_xor(ss[mt], 16, 64);
        ss[mt] = ss[mt] + __shfl_xor(ss[mt], 32, 64);
        if (cls == 0) sumsq[(wave * MT + mt) * 16 + col] = ss[mt];
      }
      if (4 * lane < 32 * U) *reinterpret_cast<float4*>(&gam[wave * 32 * U + 4 * lane]) = gl;
      __syncthreads();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        float tot = 0.f;
        for (int w = 0; w < W; ++w) tot = tot + sumsq[(w * MT + mt) * 16 + col];
        const SharedDivisor denom(sqrtf(tot / (float)a.K + a.eps));
#pragma unroll
        for (int u = 0; u < U; ++u) {
          float h[8];
          unpack8<T>(xf[mt][u], h);
          const float4 g0 = *reinterpret_cast<const float4*>(&gam[wave * 32 * U + 32 * u + 8 * cls]);
          const float4 g1 = *reinterpret_cast<const float4*>(&gam[wave * 32 * U + 32 * u + 8 * cls + 4]);
          const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = denom.divide(h[e]) * g[e];
          xf[mt][u] = pack8<T>(h);
        }
      }
    }
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
  // lane l holds out[m = l % 16][weight row 4 (l / 16) + r of the workgroup], r < 4
  float b4[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.bias && (GLU || 4 * cls < a.cols)) {
    const int brow = GLU ? (cls < 2 ? n0 + 4 * cls : a.N / 2 + n0 + 4 * (cls - 2)) : n0 + 4 * cls;
    const T* bp = reinterpret_cast<const T*>(a.bias) + brow;
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
    const int m = m0 + 16 * mt + col;
    T r4[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) r4[r] = from_float<T>(s[r] + b4[r]);
    if constexpr (GLU) {
      // classes 0, 1 hold the gate columns, classes 2, 3 the up columns that meet them 32 lanes further on
      const uint2 mine = *reinterpret_cast<const uint2*>(r4);
      uint2 other;
      other.x = (uint32_t)__shfl_xor((int)mine.x, 32, 64);
      other.y = (uint32_t)__shfl_xor((int)mine.y, 32, 64);
      if (cls < 2 && m < a.M) {
        const T* u4 = reinterpret_cast<const T*>(&other);
        T y4[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) y4[r] = silu_mul_rounded<T>(r4[r], u4[r]);
        *reinterpret_cast<uint2*>(out + (int64_t)m * (a.N / 2) + n0 + 4 * cls) = *reinterpret_cast<const uint2*>(y4);
      }
    } else {
      if (m < a.M && 4 * cls < a.cols)
        *reinterpret_cast<uint2*>(out + (int64_t)m * a.N + n0 + 4 * cls) = *reinterpret_cast<const uint2*>(r4);
    }
  }
}

// NORM variants that exist: W waves per workgroup, mt row tiles, `steps` 32-wide k steps per wave
static bool norm_fits(int W, int mt, int steps) {
  if (mt > 2 || (steps != 4 && steps != 8)) return false;
  if (steps == 8) return W == 4 || (W == 8 && mt == 1);
  return W <= 8 || mt == 1;
}

template <typename T, int W, bool NORM, bool GLU>
static int launch_linear_w(const LinearArgs& a, hipStream_t stream) {
  const int tiles = GLU ? a.N / 16 : a.N / a.cols;       // GLU: 8 gate + 8 up columns each
  const dim3 grid((unsigned)(tiles * a.row_tiles)), block(64 * W);
  const int mt = a.row_tiles > 1 ? 1 : (a.M + 15) / 16;  // row tiles per workgroup
  const int steps = a.K / W / 32;                        // 32-wide k steps per wave
  if constexpr (NORM) {
    // the wave's whole share of K in one burst, at most two row tiles; the combinations left out would not fit the
    // registers of their workgroup size
    if (!norm_fits(W, mt, steps) || tiles < (a.M < 16 * mt ? a.M : 16 * mt)) return MVLLM_ERR_UNSUPPORTED;
    if (steps == 8) {
      if constexpr (W <= 8) {
        if (mt == 1) linear_small_kernel<T, 1, 8, W, true, GLU><<<grid, block, 0, stream>>>(a);
        else if constexpr (W == 4) linear_small_kernel<T, 2, 8, W, true, GLU><<<grid, block, 0, stream>>>(a);
      }
    } else {
      if (mt == 1) linear_small_kernel<T, 1, 4, W, true, GLU><<<grid, block, 0, stream>>>(a);
      else if constexpr (W <= 8) linear_small_kernel<T, 2, 4, W, true, GLU><<<grid, block, 0, stream>>>(a);
    }
    return launch_status();
  } else {
    // loads in flight per burst: 8 steps of W and x for up to 32 rows, 4 for more (registers)
    if (mt <= 2 && steps % 8 == 0) {
      if (mt == 1) linear_small_kernel<T, 1, 8, W, false, GLU><<<grid, block, 0, stream>>>(a);
      else linear_small_kernel<T, 2, 8, W, false, GLU><<<grid, block, 0, stream>>>(a);
    } else if (steps % 4 == 0) {
      if (mt == 1) linear_small_kernel<T, 1, 4, W, false, GLU><<<grid, block, 0, stream>>>(a);
      else if (mt == 2) linear_small_kernel<T, 2, 4, W, false, GLU><<<grid, block, 0, stream>>>(a);
      else if (mt == 3) linear_small_kernel<T, 3, 4, W, false, GLU><<<grid, block, 0, stream>>>(a);
      else linear_small_kernel<T, 4, 4, W, false, GLU><<<grid, block, 0, stream>>>(a);
    } else {
      return MVLLM_ERR_UNSUPPORTED;
    }
    return launch_status();
  }
}

constexpr int kLinearNarrowCols = 8;
// columns per workgroup of the plain product: narrower tiles when 16-column tiles would leave most CUs without
// a workgroup (what a CU can keep in flight bounds its share of the weight stream)
static int linear_cols(int N, bool plain) {
  return plain && N / 16 < 128 ? kLinearNarrowCols : 16;
}

constexpr int kLinearRowTileFrom = 17;
// workgroups per column tile: from this many rows on, every 16 rows of x get a workgroup of their own (the code of
// the 16-row case, which holds few registers and asks for everything at once) instead of one workgroup that walks
// all rows; the weights are then read once from HBM and again from L2
static int linear_row_tiles(int M) {
  return M >= kLinearRowTileFrom ? (M + 15) / 16 : 1;
}

// waves per workgroup: more of them share a column tile's K when the column tiles alone give too few workgroups to
// keep the memory system busy; 12 where 16 do not divide K but 12 do, each with one burst of 256 values (K = 3072:
// the MLP's down projection)
static int linear_waves(int tiles, int K, bool plain, bool norm, int mt) {
  if (norm) {
    // a wave's share of K must be one burst of 4 or 8 steps: the fewest waves that give 1024 of them in all, else the
    // most that fit; 0 when no split does
    int best = 0;
    for (int w = 4; w <= 16; w *= 2) {
      if (K % (32 * w) != 0 || !norm_fits(w, mt, K / w / 32)) continue;
      best = w;
      if ((int64_t)tiles * w >= 1024) break;
    }
    return best;
  }
  int w = 4;
  while (w < 16 && (int64_t)tiles * w < 1024 && K % (2 * w * 128) == 0) w *= 2;
  if (plain && w == 8 && (int64_t)tiles * w < 1024 && K == 12 * 256) w = 12;
  return w;
}

template <typename T, bool NORM, bool GLU>
static int launch_linear_small(const LinearArgs& a, hipStream_t stream) {
  switch (linear_waves((GLU ? a.N / 16 : a.N / a.cols) * a.row_tiles, a.K, !NORM && !GLU, NORM,
                       a.row_tiles > 1 ? 1 : (a.M + 15) / 16)) {
    case 0: return MVLLM_ERR_UNSUPPORTED;
    case 4: return launch_linear_w<T, 4, NORM, GLU>(a, stream);
    case 8: return launch_linear_w<T, 8, NORM, GLU>(a, stream);
    case 12:
      if constexpr (!NORM && !GLU) return launch_linear_w<T, 12, false, false>(a, stream);
      else return MVLLM_ERR_UNSUPPORTED;
    default: return launch_linear_w<T, 16, NORM, GLU>(a, stream);
  }
}

template <typename T>
static int launch_linear_fused(const LinearArgs& a, bool glu, hipStream_t stream) {
  if (a.gamma) return glu ? launch_linear_small<T, true, true>(a, stream) : launch_linear_small<T, true, false>(a, stream);
  return glu ? launch_linear_small<T, false, true>(a, stream) : launch_linear_small<T, false, false>(a, stream);
}

static int linear_check(const void* out, const void* x, const void* w, const void* bias, int64_t x_row_stride, int M,
                        int N, int K, int dtype) {
  if (dtype != MVLLM_BF16 && dtype != MVLLM_F16) return dtype_size(dtype) == 0 ? MVLLM_ERR_BAD_DTYPE : MVLLM_ERR_UNSUPPORTED;
  if (M < 0 || N <= 0 || K <= 0 || x_row_stride < K) return MVLLM_ERR_BAD_SHAPE;
  if (M == 0) return MVLLM_OK;
  if (!out || !x || !w) return MVLLM_ERR_NULL_POINTER;
  if (M > 64 || N % 16 != 0 || K % 512 != 0 || x_row_stride % 8 != 0) return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(x) || !aligned16(w) || (reinterpret_cast<uintptr_t>(out) & 7u) || (reinterpret_cast<uintptr_t>(bias) & 7u))
    return MVLLM_ERR_MISALIGNED;
  return MVLLM_OK;
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_linear_small_m(void* out, const void* x, const void* w, const void* bias, int64_t x_row_stride,
                                    int M, int N, int K, int dtype, void* stream) {
  const int bad = linear_check(out, x, w, bias, x_row_stride, M, N, K, dtype);
  if (bad || M == 0) return bad;
  LinearArgs a{};
  a.out = out; a.x = x; a.w = w; a.bias = bias; a.x_row_stride = x_row_stride; a.M = M; a.N = N; a.K = K;
  a.cols = linear_cols(N, true);
  a.row_tiles = linear_row_tiles(M);
  return dtype == MVLLM_BF16 ? launch_linear_fused<bf16_t>(a, false, (hipStream_t)stream)
                             : launch_linear_fused<f16_t>(a, false, (hipStream_t)stream);
}

extern "C" int mvllm_linear_small_m_plan(int M, int N, int K, int norm, int glu, int dtype, int* waves) {
  if (dtype != MVLLM_BF16 && dtype != MVLLM_F16) return dtype_size(dtype) == 0 ? MVLLM_ERR_BAD_DTYPE : MVLLM_ERR_UNSUPPORTED;
  if (M <= 0 || N <= 0 || K <= 0) return MVLLM_ERR_BAD_SHAPE;
  if (M > 64 || N % 16 != 0 || K % 512 != 0 || (glu && N % 32 != 0)) return MVLLM_ERR_UNSUPPORTED;
  const int rt = linear_row_tiles(M), mt = rt > 1 ? 1 : (M + 15) / 16;
  const int w = linear_waves(N / linear_cols(N, !norm && !glu) * rt, K, !norm && !glu, norm != 0, mt);
  if (w == 0) return MVLLM_ERR_UNSUPPORTED;
  const int steps = K / w / 32;
  if (norm ? (!norm_fits(w, mt, steps) || N / 16 < (M < 16 * mt ? M : 16 * mt)) : (steps % 4 != 0)) return MVLLM_ERR_UNSUPPORTED;
  if (waves) *waves = w;
  return MVLLM_OK;
}

extern "C" int mvllm_norm_linear_small_m(void* out, void* residual_out, const void* x, const void* residual,
                                         const float* gamma, float eps, const void* w, const void* bias,
                                         int64_t x_row_stride, int M, int N, int K, int glu, int dtype, void* stream) {
  const int bad = linear_check(out, x, w, bias, x_row_stride, M, N, K, dtype);
  if (bad || M == 0) return bad;
  if (glu && N % 32 != 0) return MVLLM_ERR_UNSUPPORTED;
  if ((residual || residual_out) && !gamma) return MVLLM_ERR_NULL_POINTER;
  if (gamma) {
    if (!aligned16(gamma) || (residual && !aligned16(residual)) || (residual_out && !aligned16(residual_out)))
      return MVLLM_ERR_MISALIGNED;
    if (residual_out && (residual_out == x || residual_out == residual)) return MVLLM_ERR_BAD_SHAPE;
  }
  LinearArgs a{};
  a.out = out; a.x = x; a.w = w; a.bias = bias; a.x_row_stride = x_row_stride; a.M = M; a.N = N; a.K = K;
  a.residual = residual; a.residual_out = residual_out; a.gamma = gamma; a.eps = eps;
  a.cols = linear_cols(N, !gamma && !glu);
  a.row_tiles = linear_row_tiles(M);
  return dtype == MVLLM_BF16 ? launch_linear_fused<bf16_t>(a, glu != 0, (hipStream_t)stream)
                             : launch_linear_fused<f16_t>(a, glu != 0, (hipStream_t)stream);
}
