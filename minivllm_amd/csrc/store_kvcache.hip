// store_kvcache: slot_mapping scatter of K/V token rows into the paged cache,
// plain copy and per-(token, head) symmetric INT8 quantisation.
// Replaces the Triton kernel of src/myvllm/layers/attention.py:7-64.
//
// A token row (all kv heads) is Hkv*D elements, contiguous both in the input
// [T, Hkv, D] and in the flat slot view [num_slots, Hkv, D] of the cache, so
// the copy moves whole rows with the widest vector the row size allows; the
// slot index is read once per (token, thread) from L1/L2.
#include "common.h"

namespace mvllm {

constexpr int kStoreThreads = 256;

// VEC = uint4 / uint2 / uint32_t / uint16_t.  units_per_row = row bytes / sizeof(VEC).
template <typename VEC>
__global__ __launch_bounds__(kStoreThreads) void store_rows_kernel(
    const VEC* __restrict__ key, const VEC* __restrict__ value,
    VEC* __restrict__ k_cache, VEC* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping,
    int64_t num_tokens, int64_t num_slots, int units_per_row, int tokens_per_block) {
  const int64_t tok0 = (int64_t)blockIdx.x * tokens_per_block;
  const int work = tokens_per_block * units_per_row;
  for (int i = threadIdx.x; i < work; i += kStoreThreads) {
    const int tl = i / units_per_row;
    const int u = i - tl * units_per_row;
    const int64_t t = tok0 + tl;
    if (t >= num_tokens) break;
    const int64_t slot = slot_mapping[t];
    if (slot < 0 || slot >= num_slots) continue;
    const VEC kv = key[t * units_per_row + u];
    const VEC vv = value[t * units_per_row + u];
    k_cache[slot * units_per_row + u] = kv;
    v_cache[slot * units_per_row + u] = vv;
  }
}

// ---- INT8 ------------------------------------------------------------------
// GROUP lanes cooperate on one (token, kv head) vector; each lane owns 8
// consecutive elements per step.  amax by xor-shuffle inside the group (max is
// exact, so the order is irrelevant), then IEEE divide and round-half-even.
template <typename T> struct Load8;
template <> struct Load8<float> {
  static __device__ __forceinline__ void run(const float* p, float (&x)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  }
};
template <typename T16> struct Load8 {
  static __device__ __forceinline__ void run(const T16* p, float (&x)[8]) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    x[0] = lo_to_float<T16>(w.x); x[1] = hi_to_float<T16>(w.x);
    x[2] = lo_to_float<T16>(w.y); x[3] = hi_to_float<T16>(w.y);
    x[4] = lo_to_float<T16>(w.z); x[5] = hi_to_float<T16>(w.z);
    x[6] = lo_to_float<T16>(w.w); x[7] = hi_to_float<T16>(w.w);
  }
};

constexpr int kQuantMaxSteps = 4;  // head_dim <= GROUP * 8 * kQuantMaxSteps

template <typename T, int GROUP>
__device__ __forceinline__ void quantize_vector(const T* __restrict__ src, int8_t* __restrict__ dst,
                                                float* __restrict__ scale_out, int head_dim, int lane_in_group) {
  float x[kQuantMaxSteps][8];
  float amax = 0.f;
#pragma unroll
  for (int s = 0; s < kQuantMaxSteps; ++s) {
    const int e0 = (s * GROUP + lane_in_group) * 8;
    if (e0 < head_dim) {
      Load8<T>::run(src + e0, x[s]);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(x[s][j]));
    }
  }
#pragma unroll
  for (int o = GROUP / 2; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
  const float scale = amax / 127.0f;
  const bool live = scale > 0.f;
  const float div = live ? scale : 1.0f;
#pragma unroll
  for (int s = 0; s < kQuantMaxSteps; ++s) {
    const int e0 = (s * GROUP + lane_in_group) * 8;
    if (e0 < head_dim) {
      uint32_t w[2] = {0u, 0u};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float r = rintf(x[s][j] / div);
        r = fminf(fmaxf(r, -127.f), 127.f);
        const int c = live ? (int)r : 0;
        w[j >> 2] |= ((uint32_t)(c & 0xff)) << (8 * (j & 3));
      }
      *reinterpret_cast<uint2*>(dst + e0) = make_uint2(w[0], w[1]);
    }
  }
  if (lane_in_group == 0) *scale_out = scale;
}

template <typename T, int GROUP>
__global__ __launch_bounds__(kStoreThreads) void store_int8_kernel(
    const T* __restrict__ key, const T* __restrict__ value,
    int8_t* __restrict__ k_cache, int8_t* __restrict__ v_cache,
    float* __restrict__ k_scale, float* __restrict__ v_scale,
    const int64_t* __restrict__ slot_mapping,
    int64_t num_tokens, int64_t num_slots, int num_kv_heads, int head_dim) {
  constexpr int kVecPerBlock = kStoreThreads / GROUP;
  const int64_t vec = (int64_t)blockIdx.x * kVecPerBlock + threadIdx.x / GROUP;  // (token, head) index
  const int lane_in_group = threadIdx.x % GROUP;
  if (vec >= num_tokens * num_kv_heads) return;   // whole groups leave together
  const int64_t t = vec / num_kv_heads;
  const int h = (int)(vec - t * num_kv_heads);
  const int64_t slot = slot_mapping[t];
  if (slot < 0 || slot >= num_slots) return;
  const int64_t src = vec * head_dim;
  const int64_t dst = (slot * num_kv_heads + h) * head_dim;
  const int64_t sdst = slot * num_kv_heads + h;
  quantize_vector<T, GROUP>(key + src, k_cache + dst, k_scale + sdst, head_dim, lane_in_group);
  quantize_vector<T, GROUP>(value + src, v_cache + dst, v_scale + sdst, head_dim, lane_in_group);
}

template <typename T>
static int launch_store_int8(const void* key, const void* value, int8_t* k_cache, int8_t* v_cache,
                             float* k_scale, float* v_scale, const int64_t* slot_mapping,
                             int64_t num_tokens, int64_t num_slots, int num_kv_heads, int head_dim,
                             hipStream_t stream) {
  const int lanes = head_dim / 8;  // lanes needed for one pass
  const int64_t vecs = num_tokens * num_kv_heads;
#define MVLLM_LAUNCH_Q(G)                                                                              \
  do {                                                                                                 \
    const int64_t blocks = (vecs + (kStoreThreads / G) - 1) / (kStoreThreads / G);                      \
    store_int8_kernel<T, G><<<dim3((unsigned)blocks), dim3(kStoreThreads), 0, stream>>>(               \
        (const T*)key, (const T*)value, k_cache, v_cache, k_scale, v_scale, slot_mapping, num_tokens,  \
        num_slots, num_kv_heads, head_dim);                                                            \
  } while (0)
  if (lanes <= 4) MVLLM_LAUNCH_Q(4);
  else if (lanes <= 8) MVLLM_LAUNCH_Q(8);
  else if (lanes <= 16) MVLLM_LAUNCH_Q(16);
  else if (lanes <= 32) MVLLM_LAUNCH_Q(32);
  else MVLLM_LAUNCH_Q(64);
#undef MVLLM_LAUNCH_Q
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

extern "C" int mvllm_store_kvcache(const void* key, const void* value, void* k_cache, void* v_cache,
                                   const int64_t* slot_mapping, int64_t num_tokens, int64_t num_slots,
                                   int num_kv_heads, int head_dim, int dtype, void* stream) {
  const int esize = dtype_size(dtype);
  if (esize == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_tokens < 0 || num_slots < 0 || num_kv_heads <= 0 || head_dim <= 0) return MVLLM_ERR_BAD_SHAPE;
  if (num_tokens == 0) return MVLLM_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return MVLLM_ERR_NULL_POINTER;
  const int64_t row_bytes = (int64_t)num_kv_heads * head_dim * esize;
  if (row_bytes > (1 << 24)) return MVLLM_ERR_UNSUPPORTED;
  const uintptr_t all = reinterpret_cast<uintptr_t>(key) | reinterpret_cast<uintptr_t>(value) |
                        reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) |
                        (uintptr_t)row_bytes;
  hipStream_t s = (hipStream_t)stream;
#define MVLLM_LAUNCH_COPY(VEC)                                                                         \
  do {                                                                                                 \
    const int upr = (int)(row_bytes / (int64_t)sizeof(VEC));                                           \
    int tpb = (4 * kStoreThreads) / upr;                                                               \
    if (tpb < 1) tpb = 1;                                                                              \
    const int64_t blocks = (num_tokens + tpb - 1) / tpb;                                               \
    store_rows_kernel<VEC><<<dim3((unsigned)blocks), dim3(kStoreThreads), 0, s>>>(                     \
        (const VEC*)key, (const VEC*)value, (VEC*)k_cache, (VEC*)v_cache, slot_mapping, num_tokens,    \
        num_slots, upr, tpb);                                                                          \
  } while (0)
  if ((all & 15u) == 0) MVLLM_LAUNCH_COPY(uint4);
  else if ((all & 7u) == 0) MVLLM_LAUNCH_COPY(uint2);
  else if ((all & 3u) == 0) MVLLM_LAUNCH_COPY(uint32_t);
  else MVLLM_LAUNCH_COPY(uint16_t);
#undef MVLLM_LAUNCH_COPY
  return launch_status();
}

extern "C" int mvllm_store_kvcache_int8(const void* key, const void* value, int8_t* k_cache, int8_t* v_cache,
                                        float* k_scale, float* v_scale, const int64_t* slot_mapping,
                                        int64_t num_tokens, int64_t num_slots, int num_kv_heads, int head_dim,
                                        int dtype, void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_tokens < 0 || num_slots < 0 || num_kv_heads <= 0 || head_dim <= 0) return MVLLM_ERR_BAD_SHAPE;
  if (head_dim % 8 != 0 || head_dim > 64 * 8 * kQuantMaxSteps) return MVLLM_ERR_UNSUPPORTED;
  if (num_tokens == 0) return MVLLM_OK;
  if (!key || !value || !k_cache || !v_cache || !k_scale || !v_scale || !slot_mapping) return MVLLM_ERR_NULL_POINTER;
  if (!aligned16(key) || !aligned16(value) || !aligned16(k_cache) || !aligned16(v_cache)) return MVLLM_ERR_MISALIGNED;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MVLLM_F32:
      return launch_store_int8<float>(key, value, k_cache, v_cache, k_scale, v_scale, slot_mapping, num_tokens,
                                      num_slots, num_kv_heads, head_dim, s);
    case MVLLM_BF16:
      return launch_store_int8<bf16_t>(key, value, k_cache, v_cache, k_scale, v_scale, slot_mapping, num_tokens,
                                       num_slots, num_kv_heads, head_dim, s);
    default:
      return launch_store_int8<f16_t>(key, value, k_cache, v_cache, k_scale, v_scale, slot_mapping, num_tokens,
                                      num_slots, num_kv_heads, head_dim, s);
  }
}
