// mvllm_qk_norm_rope_store: everything the caller does between the QKV projection and the attention kernels,
// in one launch.  Replaces the chain Qwen3Attention.forward runs per layer and step
// (src/myvllm/models/qwen3.py:90-110):
//   q = rms_norm(q); k = rms_norm(k)        layers/layernorm.py:9-17   (one gamma over head_dim, shared by q and k)
//   q, k = rotary_emb(positions, q, k)      layers/rotary_embedding.py:4-23, 77-83   (half-split rotation)
//   store_kvcache(k, v, k_cache, v_cache, slot_mapping)   layers/attention.py:67-108
// Rounding follows that chain: the norm result is rounded to the element type, the rotation is computed in fp32
// from the rounded values and rounded again; products and sums are separate IEEE operations (no fused
// multiply-add), division and square root are correctly rounded.  Only the order of the sum of squares is free.
//
// Work item = one (token, head) vector of q, k or v.  GROUP = head_dim / 8 lanes (next power of two) share a
// vector; lane j holds elements [4j, 4j+4) of the first half and the same four of the second half, i.e.
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

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  }
};
template <typename T16> struct Vec4 {
  static __device__ __forceinline__ void load(const T16* p, float (&x)[4]) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    x[0] = lo_to_float<T16>(w.x); x[1] = hi_to_float<T16>(w.x);
    x[2] = lo_to_float<T16>(w.y); x[3] = hi_to_float<T16>(w.y);
  }
  static __device__ __forceinline__ void store(T16* p, const float (&x)[4]) {
    T16 o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = from_float<T16>(x[e]);
    *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(o);
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

__device__ __forceinline__ uint32_t pack_codes(const float (&x)[4], float div, bool live) {
  uint32_t w = 0u;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r = rintf(x[e] / div);
    r = fminf(fmaxf(r, -127.f), 127.f);
    const int c = live ? (int)r : 0;
    w |= ((uint32_t)(c & 0xff)) << (8 * e);
  }
  return w;
}

constexpr int kFusedThreads = 256;

template <typename T, int GROUP, bool INT8>
__global__ __launch_bounds__(kFusedThreads) void qk_norm_rope_store_kernel(const FusedArgs a) {
  constexpr int kVecPerBlock = kFusedThreads / GROUP;
  const int j = threadIdx.x % GROUP;
  const int per_token = a.num_heads + 2 * a.num_kv_heads;
  const int64_t item = (int64_t)blockIdx.x * kVecPerBlock + threadIdx.x / GROUP;
  if (item >= a.num_tokens * per_token) return;          // whole groups leave together
  const int64_t t = item / per_token;
  const int i = (int)(item - t * per_token);
  const int D = a.head_dim, half = D >> 1;
  const bool lane_live = 8 * j < D;                      // GROUP may exceed head_dim / 8
  const int e1 = 4 * j, e2 = half + 4 * j;

  const int kind = i < a.num_heads ? 0 : (i < a.num_heads + a.num_kv_heads ? 1 : 2);   // q, k, v
  const int h = kind == 0 ? i : (kind == 1 ? i - a.num_heads : i - a.num_heads - a.num_kv_heads);
  const T* src = kind == 0   ? reinterpret_cast<const T*>(a.q) + t * a.q_stride
                 : kind == 1 ? reinterpret_cast<const T*>(a.k) + t * a.k_stride
                             : reinterpret_cast<const T*>(a.v) + t * a.v_stride;
  src += (int64_t)h * D;

  float x1[4] = {0.f, 0.f, 0.f, 0.f}, x2[4] = {0.f, 0.f, 0.f, 0.f};
  if (lane_live) {
    Vec4<T>::load(src + e1, x1);
    Vec4<T>::load(src + e2, x2);
  }

  if (kind != 2) {
    if (a.gamma) {
      // x / sqrt(mean(x^2) + eps) * gamma, rounded to T  (layernorm.py:13-15)
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) ss = ss + x1[e] * x1[e];
#pragma unroll
      for (int e = 0; e < 4; ++e) ss = ss + x2[e] * x2[e];
      ss = group_sum<GROUP>(ss);
      const float denom = sqrtf(ss / (float)D + a.eps);
      if (lane_live) {
        float g1[4], g2[4];
        Vec4<float>::load(a.gamma + e1, g1);
        Vec4<float>::load(a.gamma + e2, g2);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x1[e] = rounded<T>((x1[e] / denom) * g1[e]);
          x2[e] = rounded<T>((x2[e] / denom) * g2[e]);
        }
      }
    }
    // out1 = x1 cos - x2 sin, out2 = x1 sin + x2 cos  (rotary_embedding.py:14-22)
    if (lane_live) {
      int64_t pos = a.positions[t];
      pos = pos < 0 ? 0 : (pos >= a.max_position ? a.max_position - 1 : pos);
      float c[4], s[4];
      Vec4<float>::load(a.cos_sin + pos * D + e1, c);
      Vec4<float>::load(a.cos_sin + pos * D + e2, s);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
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
    Vec4<T>::store(dst + e1, x1);
    Vec4<T>::store(dst + e2, x2);
  }
  if (kind == 0 || !a.slot_mapping) return;

  // cache write, same slot arithmetic and skip rule as store_kvcache (attention.py:25-64)
  const int64_t slot = a.slot_mapping[t];
  if (slot < 0 || slot >= a.num_slots) return;
  const int64_t vec = slot * a.num_kv_heads + h;
  if constexpr (INT8) {
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) amax = fmaxf(amax, fmaxf(fabsf(x1[e]), fabsf(x2[e])));
    amax = group_max<GROUP>(amax);
    const float scale = amax / 127.0f;
    const bool live = scale > 0.f;
    const float div = live ? scale : 1.0f;
    int8_t* dst = reinterpret_cast<int8_t*>(kind == 1 ? a.k_cache : a.v_cache) + vec * D;
    if (lane_live) {
      *reinterpret_cast<uint32_t*>(dst + e1) = pack_codes(x1, div, live);
      *reinterpret_cast<uint32_t*>(dst + e2) = pack_codes(x2, div, live);
    }
    if (j == 0) (kind == 1 ? a.k_scale : a.v_scale)[vec] = scale;
  } else {
    if (lane_live) {
      T* dst = reinterpret_cast<T*>(kind == 1 ? a.k_cache : a.v_cache) + vec * D;
      Vec4<T>::store(dst + e1, x1);
      Vec4<T>::store(dst + e2, x2);
    }
  }
}

template <typename T>
static int launch_fused(const FusedArgs& a, bool int8, hipStream_t stream) {
  const int lanes = a.head_dim / 8;
  const int64_t vecs = a.num_tokens * (a.num_heads + 2 * a.num_kv_heads);
#define MVLLM_LAUNCH_F(G)                                                                          \
  do {                                                                                             \
    const int64_t blocks = (vecs + (kFusedThreads / G) - 1) / (kFusedThreads / G);                  \
    if (int8) qk_norm_rope_store_kernel<T, G, true><<<dim3((unsigned)blocks), dim3(kFusedThreads), 0, stream>>>(a);  \
    else qk_norm_rope_store_kernel<T, G, false><<<dim3((unsigned)blocks), dim3(kFusedThreads), 0, stream>>>(a);      \
  } while (0)
  if (lanes <= 4) MVLLM_LAUNCH_F(4);
  else if (lanes <= 8) MVLLM_LAUNCH_F(8);
  else if (lanes <= 16) MVLLM_LAUNCH_F(16);
  else if (lanes <= 32) MVLLM_LAUNCH_F(32);
  else MVLLM_LAUNCH_F(64);
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
  // every lane moves 4 elements at a time: 8-byte (16-bit types) or 16-byte (fp32) accesses
  const uintptr_t amask = esize == 4 ? 15u : 7u;
  const uintptr_t ptrs = reinterpret_cast<uintptr_t>(q_out) | reinterpret_cast<uintptr_t>(k_out) |
                         reinterpret_cast<uintptr_t>(v_out) | reinterpret_cast<uintptr_t>(q) |
                         reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                         (slot_mapping ? reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) : 0);
  if ((ptrs & amask) != 0 || !aligned16(cos_sin_cache) || (gamma && !aligned16(gamma))) return MVLLM_ERR_MISALIGNED;
  if (((q_row_stride | k_row_stride | v_row_stride) & 3) != 0) return MVLLM_ERR_MISALIGNED;

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
    case MVLLM_F32: return launch_fused<float>(a, int8, s);
    case MVLLM_BF16: return launch_fused<bf16_t>(a, int8, s);
    default: return launch_fused<f16_t>(a, int8, s);
  }
}
