// mvllm_qk_norm_rope_store: everything the caller does between the QKV projection and the attention kernels,
// in one launch.  Replaces the chain Qwen3Attention.forward runs per layer and step
// (src/myvllm/models/qwen3.py:90-110):
//   q = rms_norm(q); k = rms_norm(k)        layers/layernorm.py:9-17   (one gamma over head_dim, shared by q and k)
//   q, k = rotary_emb(positions, q, k)      layers/rotary_embedding.py:4-23, 77-83   (half-split rotation)
//   store_kvcache(k, v, k_cache, v_cache, slot_mapping)   layers/attention.py:67-108
// Rounding follows that chain: the norm result is rounded to the element type, the rotation is computed in fp32
// from the rounded values and rounded again; products and sums are separate IEEE operations (no fused
// multiply-add), the square root is correctly rounded and x / denominator is taken with one correction step from
// the correctly rounded reciprocal (SharedDivisor).  Only the order of the sum of squares is free.
//
// Work item = one (token, head) vector of q, k or v.  GROUP lanes (a power of two) share a vector; lane j holds
// EPL = 8 (4 when head_dim is not a multiple of 16) elements [EPL j, EPL j + EPL) of the first half and the same of the second half, i.e.
// exactly the pairs the rotation mixes, so the rotation needs no cross-lane traffic; the sum of squares and the
// INT8 amax are xor-shuffle reductions inside the group.
#include "common.h"

// Products and sums below must round separately, as the chain of tensor operations they restate does: no
// contraction into fused multiply-adds anywhere in this file.
#pragma clang fp contract(off)

namespace mvllm {

struct FusedArgs {
  void* q_out;
  void* k_out;
  void* v_out;
  const void* q;
  const void* k;
  const void* v;
  int64_t q_stride, k_stride, v_stride;   // elements between consecutive token rows of the inputs
  const float* gamma;                     // [head_dim] or null: no norm
  float eps;
  const float* cos_sin;                   // [max_position, head_dim]: cos (head_dim/2) | sin (head_dim/2)
  int64_t max_position;
  const int64_t* positions;
  const int64_t* slot_mapping;            // null: nothing is stored
  void* k_cache;
  void* v_cache;
  float* k_scale;
  float* v_scale;
  int64_t num_tokens, num_slots;
  int num_heads, num_kv_heads, head_dim;
};

// N = 4 or 8 consecutive elements of T <-> fp32 registers, as one 8- or 16-byte access (16 / 32 for fp32)
template <typename T, int N> struct VecN;
template <int N> struct VecN<float, N> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[N]) {
#pragma unroll
    for (int i = 0; i < N; i += 4) {
      const float4 v = *reinterpret_cast<const float4*>(p + i);
      x[i] = v.x; x[i + 1] = v.y; x[i + 2] = v.z; x[i + 3] = v.w;
    }
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[N]) {
#pragma unroll
    for (int i = 0; i < N; i += 4)
      store16_stream(p + i, make_uint4(__float_as_uint(x[i]), __float_as_uint(x[i + 1]), __float_as_uint(x[i + 2]),
                                       __float_as_uint(x[i + 3])));
  }
};
template <typename T16, int N> struct VecN {
  static __device__ __forceinline__ void load(const T16* p, float (&x)[N]) {
    uint32_t w[N / 2];
    if constexpr (N == 8) {
      const uint4 v = *reinterpret_cast<const uint4*>(p);
      w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    } else {
      const uint2 v = *reinterpret_cast<const uint2*>(p);
      w[0] = v.x; w[1] = v.y;
    }
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
      x[2 * i] = lo_to_float<T16>(w[i]);
      x[2 * i + 1] = hi_to_float<T16>(w[i]);
    }
  }
  static __device__ __forceinline__ void store(T16* p, const float (&x)[N]) {
    T16 o[N];
#pragma unroll
    for (int e = 0; e < N; ++e) o[e] = from_float<T16>(x[e]);
    if constexpr (N == 8) store16_stream(p, *reinterpret_cast<const uint4*>(o));
    else store8_stream(p, *reinterpret_cast<const uint2*>(o));
  }
};

// value after a round trip through the element type
template <typename T> __device__ __forceinline__ float rounded(float x) { return to_float(from_float<T>(x)); }

template <int GROUP> __device__ __forceinline__ float group_sum(float x) {
#pragma unroll
  for (int o = GROUP / 2; o > 0; o >>= 1) x = x + __shfl_xor(x, o, 64);
  return x;
}
template <int GROUP> __device__ __forceinline__ float group_max(float x) {
#pragma unroll
  for (int o = GROUP / 2; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// four codes per 32-bit word, element order = byte order
template <int N>
__device__ __forceinline__ void store_codes(int8_t* dst, const float (&x)[N], float div, bool live) {
  uint32_t w[N / 4];
#pragma unroll
  for (int i = 0; i < N / 4; ++i) w[i] = 0u;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    float r = rintf(x[e] / div);
    r = fminf(fmaxf(r, -127.f), 127.f);
    const int c = live ? (int)r : 0;
    w[e >> 2] |= ((uint32_t)(c & 0xff)) << (8 * (e & 3));
  }
  if constexpr (N == 8) store8_stream(dst, make_uint2(w[0], w[1]));
  else store4_stream(dst, w[0]);
}

constexpr int kFusedThreads = 256;

// EPL = elements per lane and half: 8 when head_dim is a multiple of 16 (16-byte accesses), else 4.
template <typename T, int GROUP, int EPL, bool INT8>
__global__ __launch_bounds__(kFusedThreads) void qk_norm_rope_store_kernel(const FusedArgs a) {
  constexpr int kVecPerBlock = kFusedThreads / GROUP;
  const int j = threadIdx.x % GROUP;
  const int per_token = a.num_heads + 2 * a.num_kv_heads;
  const int64_t item = (int64_t)blockIdx.x * kVecPerBlock + threadIdx.x / GROUP;
  if (item >= a.num_tokens * per_token) return;          // whole groups leave together
  const int64_t t = item / per_token;
  const int i = (int)(item - t * per_token);
  const int D = a.head_dim, half = D >> 1;
  const bool lane_live = 2 * EPL * j < D;                // GROUP may exceed the lanes a vector needs
  const int e1 = EPL * j, e2 = half + EPL * j;

  const int kind = i < a.num_heads ? 0 : (i < a.num_heads + a.num_kv_heads ? 1 : 2);   // q, k, v
  const int h = kind == 0 ? i : (kind == 1 ? i - a.num_heads : i - a.num_heads - a.num_kv_heads);
  const T* src = kind == 0   ? reinterpret_cast<const T*>(a.q) + t * a.q_stride
                 : kind == 1 ? reinterpret_cast<const T*>(a.k) + t * a.k_stride
                             : reinterpret_cast<const T*>(a.v) + t * a.v_stride;
  src += (int64_t)h * D;

  float x1[EPL], x2[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) x1[e] = x2[e] = 0.f;
  if (lane_live) {
    VecN<T, EPL>::load(src + e1, x1);
    VecN<T, EPL>::load(src + e2, x2);
  }

  if (kind != 2) {
    if (a.gamma) {
      // x / sqrt(mean(x^2) + eps) * gamma, rounded to T  (layernorm.py:13-15)
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; ++e) ss = ss + x1[e] * x1[e];
#pragma unroll
      for (int e = 0; e < EPL; ++e) ss = ss + x2[e] * x2[e];
      ss = group_sum<GROUP>(ss);
      const SharedDivisor denom(sqrtf(ss / (float)D + a.eps));
      if (lane_live) {
        float g1[EPL], g2[EPL];
        VecN<float, EPL>::load(a.gamma + e1, g1);
        VecN<float, EPL>::load(a.gamma + e2, g2);
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          x1[e] = rounded<T>(denom.divide(x1[e]) * g1[e]);
          x2[e] = rounded<T>(denom.divide(x2[e]) * g2[e]);
        }
      }
    }
    // out1 = x1 cos - x2 sin, out2 = x1 sin + x2 cos  (rotary_embedding.py:14-22)
    if (lane_live) {
      int64_t pos = a.positions[t];
      pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);
      float c[EPL], s[EPL];
      VecN<float, EPL>::load(a.cos_sin + pos * D + e1, c);
      VecN<float, EPL>::load(a.cos_sin + pos * D + e2, s);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const float o1 = x1[e] * c[e] - x2[e] * s[e];
        const float o2 = x1[e] * s[e] + x2[e] * c[e];
        x1[e] = rounded<T>(o1);
        x2[e] = rounded<T>(o2);
      }
    }
  }

  // contiguous outputs for the attention kernels
  T* dense = kind == 0   ? reinterpret_cast<T*>(a.q_out)
             : kind == 1 ? reinterpret_cast<T*>(a.k_out)
                         : reinterpret_cast<T*>(a.v_out);
  if (dense && lane_live) {
    const int heads = kind == 0 ? a.num_heads : a.num_kv_heads;
    T* dst = dense + (t * heads + h) * D;
    VecN<T, EPL>::store(dst + e1, x1);
    VecN<T, EPL>::store(dst + e2, x2);
  }
  if (kind == 0 || !a.slot_mapping) return;

  // cache write, same slot arithmetic and skip rule as store_kvcache (attention.py:25-64)
  const int64_t slot = a.slot_mapping[t];
  if (slot < 0 || slot >= a.num_slots) return;
  const int64_t vec = slot * a.num_kv_heads + h;
  if constexpr (INT8) {
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < EPL; ++e) amax = fmaxf(amax, fmaxf(fabsf(x1[e]), fabsf(x2[e])));
    amax = group_max<GROUP>(amax);
    const float scale = amax / 127.0f;
    const bool live = scale > 0.f;
    const float div = live ? scale : 1.0f;
    int8_t* dst = reinterpret_cast<int8_t*>(kind == 1 ? a.k_cache : a.v_cache) + vec * D;
    if (lane_live) {
      store_codes<EPL>(dst + e1, x1, div, live);
      store_codes<EPL>(dst + e2, x2, div, live);
    }
    if (j == 0) (kind == 1 ? a.k_scale : a.v_scale)[vec] = scale;
  } else {
    if (lane_live) {
      T* dst = reinterpret_cast<T*>(kind == 1 ? a.k_cache : a.v_cache) + vec * D;
      VecN<T, EPL>::store(dst + e1, x1);
      VecN<T, EPL>::store(dst + e2, x2);
    }
  }
}

template <typename T>
static int launch_fused(const FusedArgs& a, bool int8, bool wide, hipStream_t stream) {
  const int lanes = a.head_dim / (wide ? 16 : 8);
  const int64_t vecs = a.num_tokens * (a.num_heads + 2 * a.num_kv_heads);
#define MVLLM_LAUNCH_F(G, E)                                                                       \
  do {                                                                                             \
    const int64_t blocks = (vecs + (kFusedThreads / G) - 1) / (kFusedThreads / G);                  \
    if (int8) qk_norm_rope_store_kernel<T, G, E, true><<<dim3((unsigned)blocks), dim3(kFusedThreads), 0, stream>>>(a);  \
    else qk_norm_rope_store_kernel<T, G, E, false><<<dim3((unsigned)blocks), dim3(kFusedThreads), 0, stream>>>(a);      \
  } while (0)
  if (wide) {
    if (lanes <= 4) MVLLM_LAUNCH_F(4, 8);
    else if (lanes <= 8) MVLLM_LAUNCH_F(8, 8);
    else if (lanes <= 16) MVLLM_LAUNCH_F(16, 8);
    else MVLLM_LAUNCH_F(32, 8);
  } else {
    if (lanes <= 4) MVLLM_LAUNCH_F(4, 4);
    else if (lanes <= 8) MVLLM_LAUNCH_F(8, 4);
    else if (lanes <= 16) MVLLM_LAUNCH_F(16, 4);
    else if (lanes <= 32) MVLLM_LAUNCH_F(32, 4);
    else MVLLM_LAUNCH_F(64, 4);
  }
#undef MVLLM_LAUNCH_F
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_qk_norm_rope_store(void* q_out, void* k_out, void* v_out, const void* q, const void* k,
                                        const void* v, int64_t q_row_stride, int64_t k_row_stride,
                                        int64_t v_row_stride, const float* gamma, float eps,
                                        const float* cos_sin_cache, int64_t max_position, const int64_t* positions,
                                        const int64_t* slot_mapping, void* k_cache, void* v_cache, float* k_scale,
                                        float* v_scale, int cache_is_int8, int64_t num_tokens, int64_t num_slots,
                                        int num_heads, int num_kv_heads, int head_dim, int dtype, void* stream) {
  const int esize = dtype_size(dtype);
  if (esize == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_tokens < 0 || num_slots < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || max_position <= 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (head_dim % 8 != 0 || head_dim > 512) return MVLLM_ERR_UNSUPPORTED;
  if (q_row_stride < (int64_t)num_heads * head_dim || k_row_stride < (int64_t)num_kv_heads * head_dim ||
      v_row_stride < (int64_t)num_kv_heads * head_dim)
    return MVLLM_ERR_BAD_SHAPE;
  if (num_tokens == 0) return MVLLM_OK;
  if (!q_out || !q || !k || !v || !cos_sin_cache || !positions) return MVLLM_ERR_NULL_POINTER;
  if (slot_mapping && (!k_cache || !v_cache)) return MVLLM_ERR_NULL_POINTER;
  if (slot_mapping && cache_is_int8 && (!k_scale || !v_scale)) return MVLLM_ERR_NULL_POINTER;
  // every lane moves 4 elements at a time, 8 when head_dim is a multiple of 16 and everything is 16-byte
  // aligned: 8- or 16-byte accesses for the 16-bit types, 16-byte ones for fp32
  const uintptr_t amask = esize == 4 ? 15u : 7u;
  const uintptr_t ptrs = reinterpret_cast<uintptr_t>(q_out) | reinterpret_cast<uintptr_t>(k_out) |
                         reinterpret_cast<uintptr_t>(v_out) | reinterpret_cast<uintptr_t>(q) |
                         reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                         (slot_mapping ? reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) : 0);
  if ((ptrs & amask) != 0 || !aligned16(cos_sin_cache) || (gamma && !aligned16(gamma))) return MVLLM_ERR_MISALIGNED;
  if (((q_row_stride | k_row_stride | v_row_stride) & 3) != 0) return MVLLM_ERR_MISALIGNED;
  const bool wide = head_dim % 16 == 0 && (ptrs & 15u) == 0 && ((q_row_stride | k_row_stride | v_row_stride) & 7) == 0;

  FusedArgs a;
  a.q_out = q_out; a.k_out = k_out; a.v_out = v_out;
  a.q = q; a.k = k; a.v = v;
  a.q_stride = q_row_stride; a.k_stride = k_row_stride; a.v_stride = v_row_stride;
  a.gamma = gamma; a.eps = eps;
  a.cos_sin = cos_sin_cache; a.max_position = max_position;
  a.positions = positions; a.slot_mapping = slot_mapping;
  a.k_cache = k_cache; a.v_cache = v_cache; a.k_scale = k_scale; a.v_scale = v_scale;
  a.num_tokens = num_tokens; a.num_slots = num_slots;
  a.num_heads = num_heads; a.num_kv_heads = num_kv_heads; a.head_dim = head_dim;
  hipStream_t s = (hipStream_t)stream;
  const bool int8 = slot_mapping && cache_is_int8;
  switch (dtype) {
    case MVLLM_F32: return launch_fused<float>(a, int8, wide, s);
    case MVLLM_BF16: return launch_fused<bf16_t>(a, int8, wide, s);
    default: return launch_fused<f16_t>(a, int8, wide, s);
  }
}
