// Device helpers shared by the LDS-tiled prefill kernels (prefill_varlen.hip, prefill_pingpong.hip): 16-bit packing,
// row sums on the dot unit, the lane-xor-32 maximum, and the global -> LDS copy with its buffer descriptor.
#pragma once
#include <type_traits>
#include <utility>
#include "common.h"

namespace mvllm {

typedef __attribute__((ext_vector_type(4))) short v4s;
typedef __attribute__((ext_vector_type(2))) float v2f;
typedef __attribute__((ext_vector_type(2))) __bf16 v2bf16;
typedef __attribute__((ext_vector_type(2))) _Float16 v2f16;


// v_max3_f32 without the canonicalising self-max the compiler puts in front of every fmaxf operand that
// comes out of an MFMA (scores are finite or -inf here, never NaN).  The compiler does not know what the asm
// reads, so it does not space it from an MFMA that writes an operand: the caller has to order it after an
// ordinary instruction that reads the newest MFMA result.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// max(x[l], x[l ^ 32]) in every lane l, by v_permlane32_swap.
__device__ __forceinline__ float max_with_lane_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  // r[0] = (x[0..31], x[0..31]), r[1] = (x[32..63], x[32..63]): their maximum is max(x[l], x[l ^ 32]) in every lane
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// x[l] + x[l ^ 32] in every lane l.
__device__ __forceinline__ float sum_with_lane_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Compile-time loop: f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{}).
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  v2f x = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, v2bf16));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  v2f x = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, v2f16));
}

// (lo, hi) of a packed 16-bit pair, each multiplied by c and rounded back to the element type.
template <typename T> __device__ __forceinline__ uint32_t scale_pair(uint32_t w, float c) {
  return pack2<T>(lo_to_float<T>(w) * c, hi_to_float<T>(w) * c);
}
// acc + lo + hi of a packed 16-bit pair in one instruction (v_dot2_f32_bf16 / v_dot2_f32_f16 against (1, 1)).
template <typename T> __device__ __forceinline__ float add_pair(uint32_t w, float acc);
template <> __device__ __forceinline__ float add_pair<bf16_t>(uint32_t w, float acc) {
  const v2bf16 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf16, w), ones, acc, false);
}
template <> __device__ __forceinline__ float add_pair<f16_t>(uint32_t w, float acc) {
  const v2f16 ones = {(_Float16)1.0f, (_Float16)1.0f};
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2f16, w), ones, acc, false);
}

// 16 bytes per lane from a buffer resource (wave-uniform descriptor + per-lane 32-bit byte offset) straight
// into LDS at lds_base + 16 * lane (buffer_load_dwordx4 ... lds).  Lanes whose offset is at or past the
// descriptor's size read nothing and get zeros written, so tiles that run past the end of the tensor need no
// clamping.  Written as inline asm on purpose: the compiler then neither tracks the transfer in vmcnt nor
// inserts a full vmcnt(0) wait before the next LDS read, so the copy of tile j+1 really overlaps the math on
// tile j; completion is awaited explicitly with dma_wait_all() before the barrier.  No "memory" clobber: the
// destination buffer is not touched by ordinary code until after that wait and barrier (which do clobber), and
// a clobber here would pin every LDS read of the tile in flight to its side of the copy.
typedef __attribute__((ext_vector_type(4))) int v4i;
template <int LDS_IMM>   // LDS destination = lds_base + LDS_IMM: one scalar register serves all copies of a wave
__device__ __forceinline__ void dma16_to_lds(v4i rsrc, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(lane_off), "s"(rsrc), "n"(LDS_IMM) : "scc", "m0");
}
// Raw buffer descriptor: 48-bit base, stride 0, size in bytes, 32-bit untyped data.
__device__ __forceinline__ v4i make_rsrc(const char* base, uint32_t bytes) {
  const uint64_t b = (uint64_t)base;
  v4i r;
  r[0] = (int)(uint32_t)b;
  r[1] = (int)((uint32_t)(b >> 32) & 0xffffu);
  r[2] = (int)bytes;
  r[3] = 0x00020000;
  return r;
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

}  // namespace mvllm
