// Shared device helpers for the gfx950 kernels of libminivllm_amd.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/minivllm_amd.h"

namespace mvllm {

typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;
typedef __attribute__((ext_vector_type(8))) _Float16 v8f16;
typedef __attribute__((ext_vector_type(4))) float v4f;
typedef __attribute__((ext_vector_type(16))) float v16f;

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---- element types ---------------------------------------------------------
// Storage structs so templates can be instantiated per dtype without pulling in
// the HIP bf16/half class headers.
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t x) { return (float)x.v; }

// round-to-nearest-even conversions from fp32
template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  // the hardware conversion (v_cvt_pk_bf16_f32): nearest even, NaN stays NaN; as bit arithmetic with a NaN test it
  // cost a dozen instructions and a branch per value
  bf16_t r;
  r.bits = __builtin_bit_cast(uint16_t, (__bf16)x);
  return r;
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float x) {
  f16_t r;
  r.v = (_Float16)x;
  return r;
}

// The two 16-bit halves of a 32-bit word as fp32 (bf16 / fp16 pairs).
template <typename T> __device__ __forceinline__ float lo_to_float(uint32_t w);
template <typename T> __device__ __forceinline__ float hi_to_float(uint32_t w);
template <> __device__ __forceinline__ float lo_to_float<bf16_t>(uint32_t w) { return __uint_as_float(w << 16); }
template <> __device__ __forceinline__ float hi_to_float<bf16_t>(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
template <> __device__ __forceinline__ float lo_to_float<f16_t>(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
}
template <> __device__ __forceinline__ float hi_to_float<f16_t>(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
}

// 16x16x32 MFMA on 8-element 16-bit fragments held as uint4.
template <typename T> __device__ __forceinline__ v4f mfma16x16x32(uint4 a, uint4 b, v4f c);
template <> __device__ __forceinline__ v4f mfma16x16x32<bf16_t>(uint4 a, uint4 b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf16, a), __builtin_bit_cast(v8bf16, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ v4f mfma16x16x32<f16_t>(uint4 a, uint4 b, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8f16, a), __builtin_bit_cast(v8f16, b), c, 0, 0, 0);
}

// 32x32x16 MFMA.
template <typename T> __device__ __forceinline__ v16f mfma32x32x16(uint4 a, uint4 b, v16f c);
template <> __device__ __forceinline__ v16f mfma32x32x16<bf16_t>(uint4 a, uint4 b, v16f c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf16, a), __builtin_bit_cast(v8bf16, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ v16f mfma32x32x16<f16_t>(uint4 a, uint4 b, v16f c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8f16, a), __builtin_bit_cast(v8f16, b), c, 0, 0, 0);
}

// ---- cross-lane helpers ----------------------------------------------------
// Value held by lane (quad base + SRC) of the caller's 4-lane quad.
template <int SRC> __device__ __forceinline__ float quad_bcast(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), SRC * 0x55, 0xf, 0xf, false));
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}

// 16-byte global load with the non-temporal hint: for data that is read once and should stream through the
// caches instead of displacing what is reused (K/V cache blocks in decode).  Measured on MI355X a pure read
// stream reaches about 7.1 TB/s with the hint against 6.0-6.5 TB/s without.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
__device__ __forceinline__ uint4 load16_stream(const void* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

// Global stores with the non-temporal hint, for output that nothing in the same kernel reads back (cache rows,
// the packed q/k/v a later kernel consumes): the lines are not kept in L2 at the expense of the streams being
// read.  Measured on MI355X in the q/k norm + rotary + store kernel (a 1 : 1.3 read : write mix of 474 MB):
// 4.1 -> 5.1 TB/s, and the prefill kernel that reads the outputs next is not slowed down.
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2_t;
__device__ __forceinline__ void store16_stream(void* p, uint4 v) {
  __builtin_nontemporal_store((u32x4){v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ void store8_stream(void* p, uint2 v) {
  __builtin_nontemporal_store((u32x2_t){v.x, v.y}, reinterpret_cast<u32x2_t*>(p));
}
__device__ __forceinline__ void store4_stream(void* p, uint32_t v) {
  __builtin_nontemporal_store(v, reinterpret_cast<uint32_t*>(p));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// x / d for many x and one d: r = 1 / d is computed once (correctly rounded), then each quotient costs a
// multiply and two FMAs instead of a full division sequence: q = x r, q + (x - q d) r.  With a correctly rounded
// reciprocal the corrected quotient is the correctly rounded x / d for normal operands (Markstein), up to rare
// last-bit cases.
struct SharedDivisor {
  float d, r;
  __device__ __forceinline__ explicit SharedDivisor(float divisor) : d(divisor), r(1.0f / divisor) {}
  __device__ __forceinline__ float divide(float x) const {
    const float q = x * r;
    return fmaf(fmaf(-q, d, x), r, q);
  }
};

// ---- host helpers ----------------------------------------------------------
inline int dtype_size(int dtype) {
  switch (dtype) {
    case MVLLM_F32: return 4;
    case MVLLM_BF16: return 2;
    case MVLLM_F16: return 2;
    default: return 0;
  }
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

// Tile `tile` (global numbering) -> sequence and first row inside it.  Wave-parallel: 64 sequences
// per step (tile counts, inclusive prefix sum by shuffles, ballot to pick the owner), so the cost is
// a few hundred cycles per 64 sequences instead of one dependent load per sequence.  Every lane of
// the calling wave must be active; all lanes return the same values.
__device__ __forceinline__ bool locate_tile(const int32_t* __restrict__ cu, int num_seqs, int tile, int bm,
                                            int& seq_start, int& seq_len, int& row0, int& seq_index) {
  const int lane = threadIdx.x & 63;
  int first = 0;
  for (int base = 0; base < num_seqs; base += 64) {
    const int s = base + lane;
    int lo = 0, len = 0;
    if (s < num_seqs) {
      lo = cu[s];
      len = cu[s + 1] - lo;
    }
    const int n = (len + bm - 1) / bm;
    int incl = n;                                   // inclusive prefix sum of tile counts over the lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(incl, o, 64);
      if (lane >= o) incl += t;
    }
    const int total = __shfl(incl, 63, 64);
    if (tile < first + total) {
      const unsigned long long owners = __ballot(tile < first + incl);   // first lane whose prefix passes the tile
      const int owner = __ffsll((long long)owners) - 1;
      const int start_tile = first + __shfl(incl - n, owner, 64);
      seq_start = __shfl(lo, owner, 64);
      seq_len = __shfl(len, owner, 64);
      row0 = (tile - start_tile) * bm;
      seq_index = base + owner;
      return true;
    }
    first += total;
  }
  return false;
}

// Varlen causal prefill on the decode kernel's tile arithmetic, for 16-bit head dims the LDS-tiled prefill kernel is
// not built for (head_dim 64).  Defined in paged_decode.hip, where that arithmetic lives; launched from the prefill
// entry point.
struct PrefillRowsArgs {
  void* out;
  const void* q;
  const void* k;
  const void* v;
  const int32_t* cu_seqlens;
  int64_t total_tokens;
  int num_seqs;
  int num_heads;
  int num_kv_heads;
  float scale_log2;
  // paged mode (k, v are caches [num_blocks, block_size, Hkv, D] holding every key; cu_seqlens counts the query
  // rows, cu_seqlens_k the keys): null / 0 otherwise
  const int32_t* cu_seqlens_k;
  const int32_t* block_tables;
  int max_num_blocks;
  int block_size;
  int64_t num_blocks;
  // INT8 cache (paged mode only; k, v are the int8 codes [num_blocks, block_size, Hkv, D]): fp32 scales
  // [num_blocks, block_size, Hkv], else null
  const float* k_scale;
  const float* v_scale;
};
int launch_prefill_rows16(const PrefillRowsArgs& a, int head_dim, int dtype, hipStream_t stream);
// shapes that kernel is built for: fp32 and INT8 caches with 64 or 128 dims per head, 16-bit also with 32, 80, 96, 112 and 256
bool prefill_rows16_takes(int head_dim, int dtype, bool int8_cache);

// Varlen causal prefill in the two-group form (prefill_pingpong.hip): one persistent 8-wave workgroup per CU whose two
// wave groups alternate between the matrix unit and the softmax.  Launched from the prefill entry point for the batches
// it takes; everything else stays on prefill_mfma_kernel.
struct PrefillPpArgs {
  void* out;
  const void* q;
  const void* k;
  const void* v;
  const int32_t* cu_seqlens;
  int64_t total_tokens;
  int num_seqs;
  int num_heads;
  int num_kv_heads;
  float scale_log2;
  // paged mode (block_tables != null): k, v are caches [num_blocks, block_size, Hkv, D]; q, out and cu_seqlens cover the
  // tokens after each sequence's cached prefix, cu_seqlens_k all of its keys
  const int32_t* cu_seqlens_k;
  const int32_t* block_tables;
  int max_num_blocks;
  int block_size;
  int64_t num_blocks;
  // filled in by the launcher
  unsigned block_magic;   // 2^32 / block_size + 1
  int block_bytes;        // bytes of one cache block (all kv heads); filled by the launcher
  int num_blocks32;       // num_blocks, capped at 2^31 - 1 (table entries are 32-bit); filled by the launcher
  int slices;       // head slices: kv heads x (query heads per kv head / heads per item)
  int n_teams;      // gcd(8, slices): workgroup teams, each with its own item list
  int team_size;    // workgroups per team
  int level_bits;   // bits that hold the block count of the longest possible sequence
  unsigned spt_magic, chunks_magic;   // 2^32 / d + 1 for d = slices per team and d = query heads per kv head / heads per item (0 for d = 1)
  // timing build only (the probe library): where workgroup `timeline_block` logs its clock stamps; null otherwise
  unsigned long long* timeline;
  int timeline_entries;
  int timeline_block;
};
// block_size: 0 for the packed entry point
bool prefill_pp_takes(int num_seqs, int num_heads, int num_kv_heads, int head_dim, int dtype, int block_size);
int launch_prefill_pp(const PrefillPpArgs& a, int dtype, hipStream_t stream);

}  // namespace mvllm
