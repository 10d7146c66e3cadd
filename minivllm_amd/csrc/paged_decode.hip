// Paged-attention decode for gfx950: split-K over fixed token partitions,
// GQA-shared K/V reads, log-sum-exp merge in a second pass.
// Replaces the Triton kernel of src/myvllm/layers/attention.py:283-415.
//
// Work decomposition (fast path, 16-bit cache, head_dim 128 or 64, block_size % 16 == 0)
//   workgroup = (partition p, sequence b, group of <= 4 kv heads); wave w of the
//   workgroup owns kv head g and all Hq/Hkv query heads that share it (16 of them at a time where a kv head has more:
//   head_slice), so the waves of one workgroup stream contiguous pieces of the [token, Hkv, D] rows.
//   A wave walks its partition in tiles of 16 tokens, both products on the matrix unit:
//     S[16 tok x 16 head]  = K_tile (A operand, straight from global in MFMA
//                            layout) x Q^T (B operand, column n = head n)
//     online softmax       per lane over its four tokens, base-2, lazy rescale with one
//                            maximum per head shared by the lanes that hold it
//     O[16 head x 128]    += P (the scores' own layout, packed to 16 bit) x V; V rows are
//                            loaded fully coalesced (lane l: tokens 4*(l/16)+i, dims 8*(l%16)..)
//                            and two byte permutes per product turn them into the B operand.
//   See DecodeHead for the operand layouts.
// The kernel is HBM-bound: a kernel that only issues the same loads (no arithmetic) reaches
// 6.25 TB/s on this access pattern, this one about 6.05.
#include <atomic>
#include <type_traits>
#include "common.h"

namespace mvllm {

// Tuning constants.
constexpr int kDecodeMaxParts = 32;
constexpr int kDecodePartCap = 1024;       // partitions grow to this many tokens while the grid stays large
constexpr int kDecodeMinPart = 256;
constexpr int kDecodeWavesPerEu = 2;
constexpr int kDecodeSmallPairs = 1024;    // partitions are shortened (to >= 64 tokens) while batch * partitions is below this
constexpr int kDecodeSmallGrid = 1024;     // kv heads per workgroup are reduced while the grid has fewer workgroups than this
constexpr int kDecodeI8Wpb = 4;            // INT8 kernel: 4-wave workgroups, three of which fit a CU (more waves to hide latency)
constexpr int kDecodeI8Threads = 256;
constexpr int kDecodeI8WavesPerEu = 3;
constexpr int kDecodeWpb = 4;              // waves (= kv heads) per workgroup, upper bound (8-wave workgroups: -1.5 %)
#ifndef MVLLM_DECODE_LOADS_ONLY
#define MVLLM_DECODE_LOADS_ONLY 0   // 1: measurement build for libmvllm_probe.so: the MFMA decode kernels issue their loads and
#endif                              // fold the loaded registers with xor instead of computing (results are meaningless)

constexpr int kTile = 16;                                 // tokens per MFMA tile
constexpr int kMaxParts = kDecodeMaxParts;         // split-K partitions per sequence (upper bound)
constexpr int kMinPartTokens = kDecodeMinPart;     // smallest partition
constexpr float kLazyRescale = 8.f;  // rescale accumulators only when the max grows by > 2^8

struct DecodeArgs {
  void* out;
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const float* k_scale;   // INT8 only
  const float* v_scale;   // INT8 only
  const int32_t* block_tables;
  const void* context_lens;
  float* ws_acc;          // [B, NP, Hq, D]
  float* ws_ml;           // [B, NP, Hq, 2]  (max in log2 units, sum)
  int64_t num_blocks;
  int ctx_is_i64;
  int max_num_blocks;
  int batch;
  int num_heads;
  int num_kv_heads;
  int head_dim;
  int block_size;
  int part_tokens;
  int num_parts;          // partitions per sequence in the grid / workspace
  float scale_log2;       // scale * log2(e)
  int head_chunks;        // MFMA kernels: slices of up to 16 query heads per kv head (1 unless a kv head has more than 16)
};

// The query heads one wave of the MFMA kernels works for.  A wave holds up to 16 query heads as the 16 columns of its
// matrix tiles.  With at most 16 query heads per kv head, slice s is kv head s with all of its query heads; with more, a
// kv head's query heads are split into head_chunks slices of 16 (the last may hold fewer), each of which streams the
// kv head's keys and values again.
struct HeadSlice {
  int kvh;      // kv head
  int head0;    // first query head
  int heads;    // query heads (<= 16)
};
__device__ __forceinline__ HeadSlice head_slice(const DecodeArgs& a, int s) {
  const int group = a.num_heads / a.num_kv_heads;
  if (a.head_chunks <= 1) return {s, s * group, group};
  const int kvh = s / a.head_chunks, c = s - kvh * a.head_chunks;
  return {kvh, kvh * group + 16 * c, min(16, group - 16 * c)};
}

// Partition length.  Lower bound: the smallest multiple of 256 tokens that covers the widest context with
// kMaxParts partitions.  Longer partitions amortise the per-workgroup start-up better (1024 tokens measured
// best on MI355X), so the length is doubled up to 1024 while the grid still offers at least four
// workgroups per CU.  A small batch of short contexts is the opposite case: too few (sequence, partition)
// pairs to occupy 256 CUs, each walking its tokens tile after tile at memory latency; there the length is
// halved, down to 64 tokens, until there are 1024 pairs.
__host__ __device__ inline int partition_tokens_for(int64_t max_ctx, int batch) {
  const int64_t per_part = (max_ctx + kMaxParts - 1) / kMaxParts;
  int64_t part = (per_part + kMinPartTokens - 1) / kMinPartTokens * kMinPartTokens;
  if (part < kMinPartTokens) part = kMinPartTokens;
  while (part < kDecodePartCap && (int64_t)batch * ((max_ctx + 2 * part - 1) / (2 * part)) >= 1024) part *= 2;
  while (part > 64 && part / 2 >= per_part && (int64_t)batch * ((max_ctx + part - 1) / part) < kDecodeSmallPairs) part /= 2;
  return (int)part;
}

inline int largest_divisor_le(int n, int cap) {
  for (int d = cap; d >= 1; --d)
    if (n % d == 0) return d;
  return 1;
}

// Small batches (fast path, both cache types).  The grid above needs many live (sequence, partition) pairs: when the batch
// is small it shortens the partitions, every sequence then needs the second launch that merges them, and when the
// contexts are much shorter than the block table is wide most of its workgroups are empty.  There a workgroup of
// kSplitWaves waves takes one (sequence, partition, kv head) instead and its waves split the tiles
// (decode_mfma_split_kernel); partitions are as long as still gives kSplitMinGroups workgroups, up to
// kSplitMaxPart tokens, so that at common serving shapes (64 sequences x 8 kv heads, tables 4096 tokens wide) a
// sequence is one workgroup and one launch.  It is chosen when partition_tokens_for could not reach its
// 1024-token partitions, when the one-wave-per-head grid would have fewer workgroups than the GPU has CUs, and
// for any batch when the table is at most kSplitMaxPart tokens wide (one partition, so never a second launch:
// 256 sequences of 96-352 tokens in a 4096-token table 99 -> 45 us, all of 4096 tokens 661 -> 674 us).  With wider
// tables and a large batch the first form is kept: it reads whole token rows and is up to 12 % faster when the
// contexts are long, although up to 2x slower when they are much shorter than the table is wide, which the
// host cannot know.
// The partition is never shorter than partition_tokens_for's, so a workspace sized from it is always enough.
constexpr int kSplitWaves = 4;            // 8 waves: 1-3 us slower per call except at 16 sequences (merge cost, one workgroup per CU)
constexpr int kSplitMinGroups = 512;
constexpr int kSplitMaxPart = 4096;
constexpr int kSplitOnePartCtx = 512;
inline bool split_wanted(int64_t max_ctx, int batch, int num_kv_heads, bool int8) {
  const int part = partition_tokens_for(max_ctx, batch);
  const int64_t parts = (max_ctx + part - 1) / part;
  const int wpb = largest_divisor_le(num_kv_heads, kDecodeWpb);
  const bool few_groups = (int64_t)batch * parts * (num_kv_heads / wpb) < 256;
  const bool short_parts = part < kDecodePartCap, narrow_table = max_ctx <= kSplitMaxPart;
  // INT8: a workgroup of the split form uses 4 of the 32 bytes of scales that a token's kv heads share, so with
  // many long sequences every head's workgroup fetches the scale lines again (128 sequences x 4096 tokens:
  // 218 -> 268 us, 256: 401 -> 467 us; 64: 123 -> 117 us): only up to 512 (sequence, kv head) pairs
  if (int8) return few_groups || ((short_parts || narrow_table) && (int64_t)batch * num_kv_heads <= 512);
  return few_groups || short_parts || narrow_table;
}
inline int split_partition_tokens(int64_t max_ctx, int batch, int num_kv_heads) {
  const int64_t pairs = (int64_t)batch * num_kv_heads;
  const int64_t want_parts = (kSplitMinGroups + pairs - 1) / pairs;
  int64_t part = ((max_ctx + want_parts - 1) / want_parts + 63) / 64 * 64;
  // a table of at most 512 tokens is one partition whatever the batch: four waves walk it in a few tiles each, and
  // the merge launch that several partitions need costs more than they save (16 sequences of 32-352 tokens:
  // 10.1 -> 8.0 us per call; from 1024-token tables on the finer split wins)
  if (max_ctx <= kSplitOnePartCtx) part = (max_ctx + 63) / 64 * 64;
  if (part > kSplitMaxPart) part = kSplitMaxPart;
  const int64_t floor_part = partition_tokens_for(max_ctx, batch);
  return (int)(part < floor_part ? floor_part : part);
}

__device__ __forceinline__ int64_t load_ctx(const DecodeArgs& a, int b) {
  int64_t c = a.ctx_is_i64 ? reinterpret_cast<const int64_t*>(a.context_lens)[b]
                           : (int64_t) reinterpret_cast<const int32_t*>(a.context_lens)[b];
  const int64_t cap = (int64_t)a.max_num_blocks * a.block_size;
  if (c > cap) c = cap;   // tokens past the table contribute nothing
  if (c < 0) c = 0;
  return c;
}

__device__ __forceinline__ float safe_exp2_diff(float m_old, float m_new) {
  // exp2(m_old - m_new) with -inf - -inf := 0 contribution
  return (m_old == -INFINITY) ? 0.f : fast_exp2(m_old - m_new);
}

// (sequence, partition) of this workgroup.  The partition index is rotated by the sequence index:
// workgroups are dealt to the 8 XCDs round-robin by linear id, and without the rotation every short
// sequence (only partition 0 live) would land on the same XCD.
//
// Order of the grid.  16-bit cache: (partition, sequence, head group), fastest first.  INT8 cache: (partition,
// head group, sequence), so that the workgroups that share a token's scales (fp32 per kv head, 32 bytes per token
// for 8 heads: every head group reads from the same 128-byte lines) run at the same time and the lines are
// fetched from memory once; with the head group slowest they were fetched once per head group (12 % of the
// kernel's time at 128 sequences, 8 kv heads in two groups).  The 16-bit kernel runs equally fast in both orders.
template <bool kSequenceSlowest>
__device__ __forceinline__ bool decode_item(const DecodeArgs& a, int& b, int& p, int& hg) {
  b = kSequenceSlowest ? blockIdx.z : blockIdx.y;
  hg = kSequenceSlowest ? blockIdx.y : blockIdx.z;
  p = (int)((blockIdx.x + (unsigned)b) % (unsigned)a.num_parts);
  return true;
}

// ---------------------------------------------------------------------------
// Fast path
// ---------------------------------------------------------------------------
// head dims of the 16-bit kernels: 32, 64, 96, 128 (one set of up to sixteen 8-dim output columns) and 256 (two sets)
constexpr int dim_sets(int d) { return d > 128 ? d / 128 : 1; }
template <typename T, int D = 128>
struct KVTile {          // 16-bit elements: lane l holds 8 dims (16 B) of token l%16 per 32-dim step, and of its four V tokens
  uint4 k[D > 128 ? D / 32 : 4];
  uint4 v[4 * dim_sets(D)];     // v[4 s + i]: token i, dims 128 s + 8 (l%16) ..
  int t0;
  bool ok;
};
template <int D>
struct KVTile<float, D> {   // fp32: 4 dims (16 B) of token l%16 per 16-dim step; of each V token 4 dims per 64-dim step
  float4 k[8];
  float4 v[4][2];
  int t0;
  bool ok;
};

// How a lane's share of a tile is addressed and loaded.  kp points at (token lane%16, first dim of class lane/16),
// vp at (one of the lane's four tokens, first dim of column lane%16).
template <typename T, int D>
struct TileIO {
  static constexpr int kKLane = 8;     // dims between the classes (lane/16) of the first product
  static constexpr int kVLane = 8;     // dims per column (lane%16) of the second product
  static constexpr int kSets = dim_sets(D);
  static __device__ __forceinline__ bool owns(int col) { return D >= 128 || col < D / 8; }
  static constexpr int kSteps = (D + 31) / 32;   // 32-dim steps of the first product; the last one may be partial
  // cls = lane / 16: the lane's 8 dims inside a step.  Head dims that are not a multiple of 32 (80, 112): the classes
  // of the last step that lie past the row's end load nothing (the next head's values are not this head's zeros).
  static __device__ __forceinline__ bool has_dims(int j, int cls) { return D % 32 == 0 || 32 * j + 8 * cls < D; }
  static __device__ __forceinline__ void load_k(KVTile<T, D>& t, const T* kp, int cls) {
#pragma unroll
    for (int j = 0; j < kSteps; ++j)
      t.k[j] = has_dims(j, cls) ? *reinterpret_cast<const uint4*>(kp + 32 * j) : make_uint4(0u, 0u, 0u, 0u);
  }
  template <bool STREAM>
  static __device__ __forceinline__ void load_v(KVTile<T, D>& t, int i, const T* vp, bool own) {
#pragma unroll
    for (int s = 0; s < kSets; ++s)
      t.v[4 * s + i] = !own ? make_uint4(0u, 0u, 0u, 0u)
                            : STREAM ? load16_stream(vp + 128 * s) : *reinterpret_cast<const uint4*>(vp + 128 * s);
  }
  static __device__ __forceinline__ void zero(KVTile<T, D>& t) {
#pragma unroll
    for (int j = 0; j < kSteps; ++j) t.k[j] = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int i = 0; i < 4 * kSets; ++i) t.v[i] = make_uint4(0u, 0u, 0u, 0u);
  }
};
template <int D>
struct TileIO<float, D> {
  static constexpr int kKLane = 4;
  static constexpr int kVLane = 4;
  static __device__ __forceinline__ bool owns(int) { return true; }     // 16 columns x 4 dims per 64-dim step
  static __device__ __forceinline__ void load_k(KVTile<float, D>& t, const float* kp, int /*cls*/) {
#pragma unroll
    for (int j = 0; j < D / 16; ++j) t.k[j] = *reinterpret_cast<const float4*>(kp + 16 * j);
  }
  template <bool STREAM>
  static __device__ __forceinline__ void load_v(KVTile<float, D>& t, int i, const float* vp, bool) {
#pragma unroll
    for (int jj = 0; jj < D / 64; ++jj) {
      if (STREAM) {
        const uint4 x = load16_stream(vp + 64 * jj);
        t.v[i][jj] = make_float4(__uint_as_float(x.x), __uint_as_float(x.y), __uint_as_float(x.z), __uint_as_float(x.w));
      } else {
        t.v[i][jj] = *reinterpret_cast<const float4*>(vp + 64 * jj);
      }
    }
  }
  static __device__ __forceinline__ void zero(KVTile<float, D>& t) {
#pragma unroll
    for (int j = 0; j < D / 16; ++j) t.k[j] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int jj = 0; jj < D / 64; ++jj) t.v[i][jj] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
};

// 16-bit pair (a, b) in the element type
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float x, float y) {
  T v[2] = {from_float<T>(x), from_float<T>(y)};
  return __builtin_bit_cast(uint32_t, v);
}
typedef __attribute__((ext_vector_type(4))) short v4i16;
typedef __attribute__((ext_vector_type(4))) _Float16 v4f16;
// D[16x16] += A[16x16] B[16x16], four 16-bit k-values per lane
template <typename T> __device__ __forceinline__ v4f mfma16x16x16(uint2 x, uint2 y, v4f c);
template <> __device__ __forceinline__ v4f mfma16x16x16<bf16_t>(uint2 x, uint2 y, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4i16, x), __builtin_bit_cast(v4i16, y), c, 0, 0, 0);
}
template <> __device__ __forceinline__ v4f mfma16x16x16<f16_t>(uint2 x, uint2 y, v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4f16, x), __builtin_bit_cast(v4f16, y), c, 0, 0, 0);
}

// Shared by the 16-bit and fp32 heads (HEAD has m, l, o[kAcc], write_row, write_partial).
template <typename HEAD>
__device__ __forceinline__ void finish_head(HEAD& hd, const DecodeArgs& a, int b, int p, int head0, int group, bool direct, int lane) {
  using T = typename HEAD::Elem;
  constexpr int D = HEAD::kDim;
  const int cls = lane >> 4;
  // denominators: add the four token classes (every lane of a head then holds the head's total)
  hd.l += __shfl_xor(hd.l, 16, 64);
  hd.l += __shfl_xor(hd.l, 32, 64);
  if (direct) {
    T* out = reinterpret_cast<T*>(a.out);
    const float linv = hd.l > 0.f ? 1.f / hd.l : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int h = 4 * cls + j;
      const float lj = __shfl(linv, h, 64);               // lane h (class 0) holds head h
      if (h < group) hd.write_row(out + ((int64_t)b * a.num_heads + head0 + h) * D, j, lj, lane);
    }
  } else {
    const int64_t slot = ((int64_t)b * a.num_parts + p) * a.num_heads + head0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int h = 4 * cls + j;
      if (h < group) hd.write_partial(a.ws_acc + (slot + h) * D, j, lane);
    }
    if (lane < group && lane < 16) *reinterpret_cast<float2*>(a.ws_ml + (slot + lane) * 2) = make_float2(hd.m, hd.l);
  }
}

// One wave = one kv head of one (sequence, partition); both products run on the matrix unit.
//   S[token][head] = K Q^T   v_mfma 16x16x32: A = 16 tokens x 32 dims (lane l: token l%16, dims 8*(l/16).. of each
//                    32-dim step, 16 B straight from the cache row), B = the query heads of the group as columns
//                    (column n = head n, zero past the group), four steps for 128 dims.  Lane l then holds
//                    S[token 4*(l/16)+i][head l%16], i < 4.
//   softmax          per lane over its four tokens; the running maximum m of a head is kept identical in the four
//                    lanes (token classes) that hold the head, so it is only exchanged when a tile raises it by
//                    more than 2^8 (lazy rescale), which is rare.
//   O[head][dim] += P V   v_mfma 16x16x16: A = P with exactly the layout S came out in (row = head l%16,
//                    k = tokens 4*(l/16)+i), packed to 16 bit; B = V with k = the same four tokens and column
//                    n = one dim per lane.  A lane loads 16 B = 8 dims of each of its four tokens (whole 256-B
//                    rows per instruction), so its dim e of step e is column l%16 of the e-th product:
//                    column n of product e is dim 8 n + e, and two byte permutes per product gather the four
//                    tokens' values of that dim.  Lane l ends with O[head 4*(l/16)+j][dims 8*(l%16) + e].
// D = 128 or 64.  With 64 the first product has two steps instead of four, and of the second product's sixteen
// columns (8 dims each) only the first eight exist: lanes l%16 >= 8 load no V, hold zero accumulators and write
// nothing.
template <typename T, int D>
struct DecodeHead {
  using Elem = T;
  static constexpr int kDim = D;
  static constexpr int kSteps = (D + 31) / 32;   // 32-dim steps of the first product; the last one may be partial
  static constexpr int kSets = dim_sets(D); // sets of sixteen 8-dim output columns (2 for head_dim 256)
  static constexpr int kCols = D >= 128 ? 16 : D / 8;   // lanes (l%16) that own 8 dims of the output per set
  static constexpr int kAcc = 8 * kSets;
  uint4 qf[kSteps];           // Q fragments: B operand, column n = head n, k = 8*cls + 32 j
  float m;                    // running maximum of head `col` (log2 units), the same in its four lanes
  float l;                    // this lane's share of the head's denominator
  v4f o[kAcc];                // o[8 s + e][j] = O[head 4*cls + j][dim 128 s + 8*col + e]

  // column lane%16 of the first product is the row of D elements at `row_ptr` (zero when not live)
  __device__ __forceinline__ void load_q(const T* row_ptr, bool live, int lane) {
    const T* src = row_ptr + (lane >> 4) * 8;
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const bool has = live && TileIO<T, D>::has_dims(j, lane >> 4);
      qf[j] = has ? *reinterpret_cast<const uint4*>(src + 32 * j) : make_uint4(0u, 0u, 0u, 0u);
    }
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int e = 0; e < kAcc; ++e) o[e] = (v4f){0.f, 0.f, 0.f, 0.f};
  }
  __device__ __forceinline__ void start(const DecodeArgs& a, int b, int head0, int group, int lane) {
    const int col = lane & 15;
    const bool live = col < group;
    load_q(reinterpret_cast<const T*>(a.q) + ((int64_t)b * a.num_heads + head0 + (live ? col : 0)) * D, live, lane);
  }
  // this lane's dims of accumulator row j (head or query row 4*(lane/16) + j), scaled, into the row of D elements
  __device__ __forceinline__ void write_row(T* row_ptr, int j, float scale, int lane) const {
    const int col = lane & 15;
    if (col < kCols) {
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        T r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = from_float<T>(o[8 * s + e][j] * scale);
        *reinterpret_cast<uint4*>(row_ptr + 128 * s + col * 8) = *reinterpret_cast<const uint4*>(r);
      }
    }
  }
  __device__ __forceinline__ void write_partial(float* row_ptr, int j, int lane) const {
    const int col = lane & 15;
    if (col < kCols) {
#pragma unroll
      for (int s = 0; s < kSets; ++s) {
        float* dst = row_ptr + 128 * s + col * 8;
        *reinterpret_cast<float4*>(dst) = make_float4(o[8 * s + 0][j], o[8 * s + 1][j], o[8 * s + 2][j], o[8 * s + 3][j]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(o[8 * s + 4][j], o[8 * s + 5][j], o[8 * s + 6][j], o[8 * s + 7][j]);
      }
    }
  }

  // one tile of 16 tokens starting at token t0 of the sequence; tokens at or past part_end do not count
  // (col_end: prefill only, where column n is a query row: tokens at or past it do not count for this lane's column)
  __device__ __forceinline__ void consume(const KVTile<T, D>& t, int part_end, float scale_log2, int lane,
                                          int col_end = 0x7fffffff) {
    if constexpr (MVLLM_DECODE_LOADS_ONLY) {      // the loads of the tile and nothing else: the access pattern's ceiling
      uint32_t x = 0;
#pragma unroll
      for (int j = 0; j < kSteps; ++j) x ^= t.k[j].x ^ t.k[j].y ^ t.k[j].z ^ t.k[j].w;
#pragma unroll
      for (int i = 0; i < 4 * kSets; ++i) x ^= t.v[i].x ^ t.v[i].y ^ t.v[i].z ^ t.v[i].w;
      l += __uint_as_float(x & 1u);
      return;
    }
    const int cls = lane >> 4;
    const int tok_base = t.t0 + 4 * cls;
    const bool partial = (!t.ok) || (t.t0 + kTile > part_end);
    v4f s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kSteps; ++j) s = mfma16x16x32<T>(t.k[j], qf[j], s);
    float s2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) s2[i] = s[i] * scale_log2;
    uint4 v[4 * kSets];
#pragma unroll
    for (int i = 0; i < 4 * kSets; ++i) v[i] = t.v[i];
    if (partial) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (!t.ok || tok_base + i >= part_end) {
          s2[i] = -INFINITY;
#pragma unroll
          for (int s = 0; s < kSets; ++s) v[4 * s + i] = make_uint4(0u, 0u, 0u, 0u);   // whatever lies there must not meet p = 0 as NaN or Inf
        }
    }
    if (col_end != 0x7fffffff) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (tok_base + i >= col_end) s2[i] = -INFINITY;
    }
    const float tile_max = fmaxf(fmaxf(s2[0], s2[1]), fmaxf(s2[2], s2[3]));
    const bool grow = tile_max > m + kLazyRescale || (m == -INFINITY && tile_max > -INFINITY);
    if (__any(grow)) {
      // the head's maximum over its four token classes, then one decision for all four lanes
      float mh = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
      mh = fmaxf(mh, __shfl_xor(mh, 32, 64));
      const bool grow_h = mh > m + kLazyRescale || (m == -INFINITY && mh > -INFINITY);
      const float m_new = grow_h ? mh : m;
      const float al = (m_new == m) ? 1.f : safe_exp2_diff(m, m_new);
      l *= al;
      m = m_new;
      // accumulator row j is head 4*cls + j, whose factor sits in lane 4*cls + j (any class would do)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float aj = __shfl(al, 4 * cls + j, 64);
#pragma unroll
        for (int e = 0; e < kAcc; ++e) o[e][j] *= aj;
      }
    }
    const float m_eff = (m == -INFINITY) ? 0.f : m;
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = fast_exp2(s2[i] - m_eff);
      l += pr[i];
    }
    const uint2 pa = make_uint2(pack_pair<T>(pr[0], pr[1]), pack_pair<T>(pr[2], pr[3]));
    // dim e of the lane's 8: the low or high half of component e/2 of each token's 16 bytes
#pragma unroll
    for (int s = 0; s < kSets; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
        const uint4 &v0 = v[4 * s], &v1 = v[4 * s + 1], &v2 = v[4 * s + 2], &v3 = v[4 * s + 3];
        const uint32_t c0 = e < 2 ? v0.x : e < 4 ? v0.y : e < 6 ? v0.z : v0.w;
        const uint32_t c1 = e < 2 ? v1.x : e < 4 ? v1.y : e < 6 ? v1.z : v1.w;
        const uint32_t c2 = e < 2 ? v2.x : e < 4 ? v2.y : e < 6 ? v2.z : v2.w;
        const uint32_t c3 = e < 2 ? v3.x : e < 4 ? v3.y : e < 6 ? v3.z : v3.w;
        const uint2 vb = make_uint2(__builtin_amdgcn_perm(c1, c0, sel), __builtin_amdgcn_perm(c3, c2, sel));
        o[8 * s + e] = mfma16x16x16<T>(pa, vb, o[8 * s + e]);
      }
  }

  // W waves hold partial results of the same heads over different tokens: waves 1 .. W-1 leave theirs in LDS
  // (1 + kAcc float4 per lane: m, l and the accumulators), wave 0 folds them into its own with the usual
  // log-sum-exp weights and is the only one to return true.  Every wave of the workgroup must call this.
  template <int W>
  __device__ __forceinline__ bool merge(int w, int lane) {
    constexpr int kSlots = 1 + kAcc;
    __shared__ float4 part[(W - 1) * kSlots * 64];
    const int cls = lane >> 4;
    if (w > 0) {
      float4* dst = part + (w - 1) * kSlots * 64 + lane;
      dst[0] = make_float4(m, l, 0.f, 0.f);
#pragma unroll
      for (int e = 0; e < kAcc; ++e) dst[(1 + e) * 64] = make_float4(o[e][0], o[e][1], o[e][2], o[e][3]);
    }
    __syncthreads();
    if (w > 0) return false;
#pragma unroll 1
    for (int x = 0; x < W - 1; ++x) {
      const float4* src = part + x * kSlots * 64 + lane;
      const float4 ml = src[0];
      const float m_new = fmaxf(m, ml.x);
      const float f0 = safe_exp2_diff(m, m_new);          // both are 0 while neither wave has seen a token
      const float f1 = safe_exp2_diff(ml.x, m_new);
      m = m_new;
      l = l * f0 + ml.y * f1;
      float a0[4], a1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {                        // accumulator row j is head 4*cls + j
        a0[j] = __shfl(f0, 4 * cls + j, 64);
        a1[j] = __shfl(f1, 4 * cls + j, 64);
      }
#pragma unroll
      for (int e = 0; e < kAcc; ++e) {
        const float4 ow = src[(1 + e) * 64];
        o[e][0] = o[e][0] * a0[0] + ow.x * a1[0];
        o[e][1] = o[e][1] * a0[1] + ow.y * a1[1];
        o[e][2] = o[e][2] * a0[2] + ow.z * a1[2];
        o[e][3] = o[e][3] * a0[3] + ow.w * a1[3];
      }
    }
    return true;
  }

  // write the output row (direct) or this partition's partial result
  __device__ __forceinline__ void finish(const DecodeArgs& a, int b, int p, int head0, int group, bool direct, int lane) {
    finish_head(*this, a, b, p, head0, group, direct, lane);
  }
};

// fp32 caches and queries: the same decomposition on v_mfma_f32_16x16x4_f32 (one fp32 value per lane and operand,
// k = lane/16), products and sums in fp32 throughout, the weights P are not rounded.
//   S[token][head]      A = K: lane l holds 4 dims (16 B) of token l%16 per 16-dim step, dims 16 j + 4 (l/16) + e;
//                       product (j, e) contracts exactly those dims; B = Q with the same dims of head l%16.
//   O[head][dim] += P V A = P as it came out (row = head l%16, k = token 4 (l/16) + i for product i); B = V: the
//                       lane's 4 dims (16 B) of that token per 64-dim step, so column n of product (i, jj, e) is dim
//                       64 jj + 4 n + e.  Lane l ends with O[head 4 (l/16) + j][dims 64 jj + 4 (l%16) + e].
template <int D>
struct DecodeHead<float, D> {
  using Elem = float;
  static constexpr int kDim = D;
  static constexpr int kSteps = D / 16;      // 16-dim steps of the first product (4 MFMAs each)
  static constexpr int kVSteps = D / 64;     // 64-dim steps of the second
  static constexpr int kAcc = 4 * kVSteps;
  float4 qf[kSteps];
  float m;
  float l;
  v4f o[kAcc];                // o[4 jj + e][j] = O[head 4*cls + j][dim 64 jj + 4 col + e]

  __device__ __forceinline__ void load_q(const float* row_ptr, bool live, int lane) {
    const float* src = row_ptr + (lane >> 4) * 4;
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const float4 x = *reinterpret_cast<const float4*>(src + 16 * j);
      qf[j] = live ? x : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int e = 0; e < kAcc; ++e) o[e] = (v4f){0.f, 0.f, 0.f, 0.f};
  }
  __device__ __forceinline__ void start(const DecodeArgs& a, int b, int head0, int group, int lane) {
    const int col = lane & 15;
    const bool live = col < group;
    load_q(reinterpret_cast<const float*>(a.q) + ((int64_t)b * a.num_heads + head0 + (live ? col : 0)) * D, live, lane);
  }

  __device__ __forceinline__ void consume(const KVTile<float, D>& t, int part_end, float scale_log2, int lane,
                                          int col_end = 0x7fffffff) {
    const int cls = lane >> 4;
    const int tok_base = t.t0 + 4 * cls;
    const bool partial = (!t.ok) || (t.t0 + kTile > part_end);
    v4f s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[j].x, qf[j].x, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[j].y, qf[j].y, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[j].z, qf[j].z, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[j].w, qf[j].w, s, 0, 0, 0);
    }
    float s2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) s2[i] = s[i] * scale_log2;
    float4 v[4][kVSteps];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int jj = 0; jj < kVSteps; ++jj) v[i][jj] = t.v[i][jj];
    if (partial) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (!t.ok || tok_base + i >= part_end) {
          s2[i] = -INFINITY;
#pragma unroll
          for (int jj = 0; jj < kVSteps; ++jj) v[i][jj] = make_float4(0.f, 0.f, 0.f, 0.f);   // must not meet p = 0 as NaN or Inf
        }
    }
    if (col_end != 0x7fffffff) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (tok_base + i >= col_end) s2[i] = -INFINITY;
    }
    const float tile_max = fmaxf(fmaxf(s2[0], s2[1]), fmaxf(s2[2], s2[3]));
    const bool grow = tile_max > m + kLazyRescale || (m == -INFINITY && tile_max > -INFINITY);
    if (__any(grow)) {
      float mh = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
      mh = fmaxf(mh, __shfl_xor(mh, 32, 64));
      const bool grow_h = mh > m + kLazyRescale || (m == -INFINITY && mh > -INFINITY);
      const float m_new = grow_h ? mh : m;
      const float al = (m_new == m) ? 1.f : safe_exp2_diff(m, m_new);
      l *= al;
      m = m_new;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float aj = __shfl(al, 4 * cls + j, 64);
#pragma unroll
        for (int e = 0; e < kAcc; ++e) o[e][j] *= aj;
      }
    }
    const float m_eff = (m == -INFINITY) ? 0.f : m;
    float pr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      pr[i] = fast_exp2(s2[i] - m_eff);
      l += pr[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int jj = 0; jj < kVSteps; ++jj) {
        o[4 * jj + 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[i], v[i][jj].x, o[4 * jj + 0], 0, 0, 0);
        o[4 * jj + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[i], v[i][jj].y, o[4 * jj + 1], 0, 0, 0);
        o[4 * jj + 2] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[i], v[i][jj].z, o[4 * jj + 2], 0, 0, 0);
        o[4 * jj + 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(pr[i], v[i][jj].w, o[4 * jj + 3], 0, 0, 0);
      }
  }

  template <int W>
  __device__ __forceinline__ bool merge(int w, int lane) {
    __shared__ float4 part[(W - 1) * (1 + kAcc) * 64];
    const int cls = lane >> 4;
    if (w > 0) {
      float4* dst = part + (w - 1) * (1 + kAcc) * 64 + lane;
      dst[0] = make_float4(m, l, 0.f, 0.f);
#pragma unroll
      for (int e = 0; e < kAcc; ++e) dst[(1 + e) * 64] = make_float4(o[e][0], o[e][1], o[e][2], o[e][3]);
    }
    __syncthreads();
    if (w > 0) return false;
#pragma unroll 1
    for (int x = 0; x < W - 1; ++x) {
      const float4* src = part + x * (1 + kAcc) * 64 + lane;
      const float4 ml = src[0];
      const float m_new = fmaxf(m, ml.x);
      const float f0 = safe_exp2_diff(m, m_new);
      const float f1 = safe_exp2_diff(ml.x, m_new);
      m = m_new;
      l = l * f0 + ml.y * f1;
      float a0[4], a1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a0[j] = __shfl(f0, 4 * cls + j, 64);
        a1[j] = __shfl(f1, 4 * cls + j, 64);
      }
#pragma unroll
      for (int e = 0; e < kAcc; ++e) {
        const float4 ow = src[(1 + e) * 64];
        o[e][0] = o[e][0] * a0[0] + ow.x * a1[0];
        o[e][1] = o[e][1] * a0[1] + ow.y * a1[1];
        o[e][2] = o[e][2] * a0[2] + ow.z * a1[2];
        o[e][3] = o[e][3] * a0[3] + ow.w * a1[3];
      }
    }
    return true;
  }

  __device__ __forceinline__ void write_row(float* row_ptr, int j, float scale, int lane) const {
    const int col = lane & 15;
#pragma unroll
    for (int jj = 0; jj < kVSteps; ++jj)
      *reinterpret_cast<float4*>(row_ptr + 64 * jj + 4 * col) =
          make_float4(o[4 * jj][j] * scale, o[4 * jj + 1][j] * scale, o[4 * jj + 2][j] * scale, o[4 * jj + 3][j] * scale);
  }
  __device__ __forceinline__ void write_partial(float* row_ptr, int j, int lane) const { write_row(row_ptr, j, 1.f, lane); }
  __device__ __forceinline__ void finish(const DecodeArgs& a, int b, int p, int head0, int group, bool direct, int lane) {
    finish_head(*this, a, b, p, head0, group, direct, lane);
  }
};

// W = 1: the wave walks all tiles of its partition.  W > 1 (the workgroup is W waves on one kv head): wave w takes
// tiles w, w + W, ... and the partial results meet in LDS (DecodeHead::merge), so a short context costs a few tiles
// of latency per wave and no second launch.
// SUB: blocks of 1, 2, 4 or 8 tokens.  A 16-token tile then spans several blocks, and every lane looks up the blocks
// of its own tokens (one for its K row, up to four for its V rows) in the block-table window.
template <typename T, int W, int D, bool SUB = false>
__device__ __forceinline__ void decode_mfma_item(const DecodeArgs& a, int b, int p, int slice, int w) {
  const int lane = threadIdx.x & 63;
  const HeadSlice hs = head_slice(a, slice);
  const int g = hs.kvh;                                // kv head
  const int group = hs.heads;                          // q heads of this wave (<= 16)
  const int col = lane & 15;                           // head (first product), dim group (second product)
  const int cls = lane >> 4;                           // token class: tokens 4*cls .. 4*cls+3 of a tile
  const int bs = a.block_size;
  const int part_start = p * a.part_tokens;
  const int first = part_start + (W == 1 ? 0 : w * kTile);      // first token of this wave's first tile
  const int32_t* table = a.block_tables + (int64_t)b * a.max_num_blocks;

  // The query rows and the block-table window (lane i holds entry win_base + i of this sequence) do not depend
  // on the context length.  The split kernel, which is all latency, asks for them together with it; the
  // one-wave form first drops the workgroups whose partition lies past the context (most of a ragged batch).
  DecodeHead<T, D> head;
  int bi = first / bs;               // logical block of the next tile to load
  int off = first - bi * bs;         // token offset inside that block
  int win_base = bi;
  int win;
  auto prologue = [&]() __attribute__((always_inline)) {
    head.start(a, b, hs.head0, group, lane);
    win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;
  };
  if constexpr (W > 1) prologue();

  const int ctx = (int)load_ctx(a, b);
  // a sequence that fits one partition (or is empty) is finished here: partition 0 writes the output row
  const bool direct = ctx <= a.part_tokens;
  if (part_start >= ctx && !(direct && p == 0)) return;
  const int part_end = min(ctx, part_start + a.part_tokens);
  const int tiles_all = part_end > part_start ? (part_end - part_start + kTile - 1) / kTile : 0;
  const int ntiles = W == 1 ? tiles_all : (tiles_all > w ? (tiles_all - w + W - 1) / W : 0);   // this wave's
  if constexpr (W == 1) prologue();

  const int64_t row = (int64_t)a.num_kv_heads * D;       // elements per token row
  const T* kc = reinterpret_cast<const T*>(a.k_cache) + (int64_t)g * D;
  const T* vc = reinterpret_cast<const T*>(a.v_cache) + (int64_t)g * D;

  using IO = TileIO<T, D>;
  const int k_lane_off = col * (int)row + cls * IO::kKLane;        // token lane%16, first dim of class lane/16
  const int v_lane_off = 4 * cls * (int)row + col * IO::kVLane;    // token 4*(lane/16), first dim of column lane%16

  auto load_tile = [&](KVTile<T, D>& t, int tile) {
    t.t0 = first + tile * (W * kTile);
    if constexpr (SUB) {
      const int lb = __builtin_ctz((unsigned)bs);              // block_size is a power of two below 16
      const int bpt = kTile >> lb;                             // blocks per tile
      if (bi + bpt - win_base > 64) {
        win_base = bi;
        win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;
      }
      // A token past the partition's end (the tile is the last one) has no block of its own: the lane loads the
      // last live token's row instead, and consume() masks it by position.
      const int live = part_end - 1 - t.t0;                    // index of the tile's last live token (>= 0)
      const int kt = col < live ? col : live;
      const int kb = bi + (kt >> lb);
      const int kphys = __shfl(win, kb - win_base, 64);
      bool ok = kb < a.max_num_blocks && kphys >= 0 && (int64_t)kphys < a.num_blocks;
      int vphys[4], vt[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vt[i] = 4 * cls + i < live ? 4 * cls + i : live;
        const int vb = bi + (vt[i] >> lb);
        vphys[i] = __shfl(win, vb - win_base, 64);
        ok = ok && vb < a.max_num_blocks && vphys[i] >= 0 && (int64_t)vphys[i] < a.num_blocks;
      }
      t.ok = __all(ok);                                        // a tile with an unmapped block is left out as a whole
      if (t.ok) {
        IO::load_k(t, kc + ((int64_t)kphys * bs + (kt & (bs - 1))) * row + cls * IO::kKLane, lane >> 4);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          IO::template load_v<true>(t, i, vc + ((int64_t)vphys[i] * bs + (vt[i] & (bs - 1))) * row + col * IO::kVLane, IO::owns(col));
      } else {
        IO::zero(t);
      }
      bi += W * bpt;
      return;
    }
    if (bi - win_base >= 64) {
      win_base = bi;
      win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;
    }
    const int phys = __builtin_amdgcn_readlane(win, bi - win_base);
    t.ok = (bi < a.max_num_blocks) && phys >= 0 && (int64_t)phys < a.num_blocks;
    if (t.ok) {
      const int64_t base = ((int64_t)phys * bs + off) * row;
      const T* kp = kc + base + k_lane_off;
      const T* vp = vc + base + v_lane_off;
      // V is read once, in whole 256-byte rows per instruction: non-temporal loads stream it past the caches.
      // K is read in the MFMA operand layout, 64 bytes of a row per instruction, so the second half of each
      // 128-byte line has to survive in cache until the next instruction: ordinary loads (the hint costs 7 %
      // there).
      IO::load_k(t, kp, lane >> 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) IO::template load_v<true>(t, i, vp + (int64_t)i * row, IO::owns(col));
    } else {
      IO::zero(t);
    }
    if constexpr (W == 1) {
      off += kTile;
      if (off >= bs) { off = 0; ++bi; }
    } else {
      off += W * kTile;
      while (off >= bs) { off -= bs; ++bi; }
    }
  };

  // Tiles in pairs (ta, tb: one consumed while the other is in flight), the odd one after the loop.  A single
  // loop exit keeps the accumulators in one set of registers (an exit between the two halves made the compiler
  // hold two: 184 VGPRs instead of 154, one wave per SIMD less).
  KVTile<T, D> ta, tb;
  if (ntiles > 0) load_tile(ta, 0);
  int tile = 0;
  for (; tile + 1 < ntiles; tile += 2) {
    load_tile(tb, tile + 1);
    head.consume(ta, part_end, a.scale_log2, lane);
    if (tile + 2 < ntiles) load_tile(ta, tile + 2);
    head.consume(tb, part_end, a.scale_log2, lane);
  }
  if (tile < ntiles) head.consume(ta, part_end, a.scale_log2, lane);
  if constexpr (W > 1) {
    if (!head.template merge<W>(w, lane)) return;
  }
  head.finish(a, b, p, hs.head0, group, direct, lane);
}

// ---------------------------------------------------------------------------
// Varlen causal prefill on the same tile arithmetic (flash_attention_prefill, attention.py:212-280), for fp32, which
// the LDS-tiled kernel of prefill_varlen.hip does not take (the reference's main.py runs in fp32).
// One wave = 16 consecutive query rows of one query head: the rows take the place of the heads of a group
// (column n of the first product = row n), the keys 0 .. row are walked in 16-token tiles straight from the
// packed k / v tensors, and the causal limit is applied per column.  The four waves of a workgroup are four query
// heads on the same rows, so with grouped heads they read the same K/V tiles at the same time.  No LDS and no
// reuse of K/V across row tiles beyond the caches: tens of TFLOP/s, not hundreds.
// ---------------------------------------------------------------------------
// PAGED: prefill of the rows that follow a cached prefix (mvllm_prefill_paged): row r of a sequence sits at key
// position cached + r and every key is read from the paged cache through the block table, as in decode.
// I8 (paged only): the cache holds int8 codes and per-(token, kv head) fp32 scales (the format store_kvcache_int8
// writes); a lane dequantises its share of a tile to the query's 16-bit type as it loads it (code * scale, rounded
// once), after which the tile is an ordinary 16-bit tile.
template <typename T>
__device__ __forceinline__ uint4 dequant8(uint2 codes, float scale) {
  const uint32_t w[2] = {codes.x, codes.y};
  uint32_t out[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float x0 = (float)(int)(int8_t)(w[e >> 1] >> (16 * (e & 1))) * scale;
    const float x1 = (float)(int)(int8_t)(w[e >> 1] >> (16 * (e & 1) + 8)) * scale;
    out[e] = pack_pair<T>(x0, x1);
  }
  return make_uint4(out[0], out[1], out[2], out[3]);
}

template <typename T, int D, bool PAGED, bool I8 = false>
__global__ __launch_bounds__(256) void prefill_rows16_kernel(const PrefillRowsArgs a, int tiles_x) {
  static_assert(!I8 || (PAGED && sizeof(T) == 2), "INT8 caches: paged mode, 16-bit queries");
  int seq_start, seq_len, row0, seq_index;
  // latest (heaviest) tiles first
  if (!locate_tile(a.cu_seqlens, a.num_seqs, tiles_x - 1 - (int)blockIdx.x, kTile, seq_start, seq_len, row0, seq_index)) return;
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, cls = lane >> 4;
  const int h = blockIdx.y * 4 + (threadIdx.x >> 6);   // query head of this wave
  if (h >= a.num_heads) return;
  const int g = h / (a.num_heads / a.num_kv_heads);
  const int rows = min(kTile, seq_len - row0);          // live query rows of the tile

  using IO = TileIO<T, D>;
  DecodeHead<T, D> head;
  {
    const bool live = col < rows;
    head.load_q(reinterpret_cast<const T*>(a.q) + ((int64_t)(seq_start + row0 + (live ? col : 0)) * a.num_heads + h) * D,
                live, lane);
  }
  const int cached = PAGED ? max(a.cu_seqlens_k[seq_index + 1] - a.cu_seqlens_k[seq_index] - seq_len, 0) : 0;
  const int kv_end = cached + row0 + rows;        // keys 0 .. kv_end - 1 are seen by at least one row of the tile
  const int col_end = cached + row0 + col + 1;    // keys seen by this lane's row
  const int ntiles = (kv_end + kTile - 1) / kTile;
  const int64_t row = (int64_t)a.num_kv_heads * D;
  const T* kc = reinterpret_cast<const T*>(a.k) + (PAGED ? 0 : (int64_t)seq_start * row) + (int64_t)g * D + cls * IO::kKLane;
  const T* vc = reinterpret_cast<const T*>(a.v) + (PAGED ? 0 : (int64_t)seq_start * row) + (int64_t)g * D + col * IO::kVLane;
  // INT8: the same element offsets in bytes
  const int8_t* kc8 = reinterpret_cast<const int8_t*>(a.k) + (int64_t)g * D + cls * 8;
  const int8_t* vc8 = reinterpret_cast<const int8_t*>(a.v) + (int64_t)g * D + col * 8;
  // paged: block-table window, lane i holds entry win_base + i of this sequence (as in the decode kernel)
  const int bs = PAGED ? a.block_size : 1;
  const int32_t* table = PAGED ? a.block_tables + (int64_t)seq_index * a.max_num_blocks : nullptr;
  int bi = 0, off = 0, win_base = 0, win = -1;
  if (PAGED) win = lane < a.max_num_blocks ? table[lane] : -1;

  // Tokens past kv_end are masked by consume(); in the packed tensors their loads are redirected to the last
  // visible row so that nothing past the end is touched (in a cache block they are rows of the same block).
  auto load_tile = [&](KVTile<T, D>& t, int tile) __attribute__((always_inline)) {
    t.t0 = tile * kTile;
    t.ok = true;
    // An unmapped block reads as zero keys and values that still count (score 0), as in the other prefill
    // kernels and unlike decode, where such tokens contribute nothing.
    bool mapped = true;
    int64_t k_tok, v_tok[4];
    if constexpr (PAGED) {
      if (bi - win_base >= 64) {
        win_base = bi;
        win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;
      }
      const int phys = __builtin_amdgcn_readlane(win, bi - win_base);
      mapped = (bi < a.max_num_blocks) && phys >= 0 && (int64_t)phys < a.num_blocks;
      const int64_t tok0 = (int64_t)(mapped ? phys : 0) * bs + off;
      k_tok = tok0 + col;
#pragma unroll
      for (int i = 0; i < 4; ++i) v_tok[i] = tok0 + 4 * cls + i;
      off += kTile;
      if (off >= bs) { off = 0; ++bi; }
    } else {
      k_tok = min(t.t0 + col, kv_end - 1);
#pragma unroll
      for (int i = 0; i < 4; ++i) v_tok[i] = min(t.t0 + 4 * cls + i, kv_end - 1);
    }
    if constexpr (I8) {
      if (mapped) {
        const float ks = a.k_scale[k_tok * a.num_kv_heads + g];
#pragma unroll
        for (int j = 0; j < D / 32; ++j) t.k[j] = dequant8<T>(*reinterpret_cast<const uint2*>(kc8 + k_tok * row + 32 * j), ks);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          t.v[i] = IO::owns(col) ? dequant8<T>(*reinterpret_cast<const uint2*>(vc8 + v_tok[i] * row),
                                               a.v_scale[v_tok[i] * a.num_kv_heads + g])
                                 : make_uint4(0u, 0u, 0u, 0u);
      } else {
        IO::zero(t);
      }
    } else if (mapped) {
      IO::load_k(t, kc + k_tok * row, lane >> 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) IO::template load_v<false>(t, i, vc + v_tok[i] * row, IO::owns(col));
    } else {
      IO::zero(t);
    }
  };
  KVTile<T, D> ta, tb;
  if (ntiles > 0) load_tile(ta, 0);
  int tile = 0;
  for (; tile + 1 < ntiles; tile += 2) {
    load_tile(tb, tile + 1);
    head.consume(ta, kv_end, a.scale_log2, lane, col_end);
    if (tile + 2 < ntiles) load_tile(ta, tile + 2);
    head.consume(tb, kv_end, a.scale_log2, lane, col_end);
  }
  if (tile < ntiles) head.consume(ta, kv_end, a.scale_log2, lane, col_end);

  // denominators over the four token classes, then row 4*cls + j of the tile, dims 8*col .. of the head
  float l = head.l;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  const float linv = l > 0.f ? 1.f / l : 0.f;
  T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = 4 * cls + j;
    const float lj = __shfl(linv, r, 64);                 // lane r (class 0) holds column r
    if (r < rows) head.write_row(out + ((int64_t)(seq_start + row0 + r) * a.num_heads + h) * D, j, lj, lane);
  }
}

// ---------------------------------------------------------------------------
// Fast path, INT8 cache (head_dim 128 or 64, block_size % 16 == 0).  Same
// decomposition as the 16-bit kernel, both products on the matrix unit.
//   QK^T   v_mfma_i32_16x16x64_i8 with the int8 codes as they lie in memory (lane = token, 16 bytes = 16 dims):
//          the query row is turned once per wave into 15-bit fixed point q ~ (128*hi + lo) * amax/16256 with
//          int8 hi/lo planes (column n = head n), so scores are exact integer dot products times
//          (amax/16256) * k_scale[token]; lane l holds S[token 4*(l/16)+r][head l%16].
//   PV     v_mfma_f32_16x16x16_f16, as in the 16-bit kernel: A = the weights p * v_scale of the lane's four
//          tokens as fp16, B = V with k = the same four tokens and column n = one dim per lane.  V rows are 128 B;
//          a lane loads 8 bytes = 8 dims of each of its four tokens (lane l: tokens 4*(l/16)+i, dims 8*(l%16)..,
//          whole rows per instruction).  The codes are biased by +128 (one xor per 4 codes) and the byte of dim e
//          of two tokens becomes the fp16 pair (1024 + u_a, 1024 + u_b) with v_perm + an or of the exponent bits
//          (0x6400 | u is exactly 1024 + u): four vector instructions per product, column n of product e is dim
//          8 n + e.  The 1024 + 128 leaves at the end as 1152 * sum(weights).  The running maximum is kept over
//          score + log2 v_scale, so weights lie in (0, 2^8] for any scales and fit fp16.
//   scales one k_scale and one v_scale load per lane and tile (lane l%4 of a quad holds token 4*(l/16)+l%4),
//          handed round inside the quad by DPP.
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) int v4i;
typedef __attribute__((ext_vector_type(2))) _Float16 v2f16;
typedef __attribute__((ext_vector_type(2))) float v2f;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

struct KVTileI8 {
  uint4 k[2];
  uint2 v[4];
  float ks;
  float vs;
  int t0;
  bool ok;
};

__device__ __forceinline__ uint2 load8_stream(const void* p) {
  const u32x2 x = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
  return make_uint2(x.x, x.y);
}

// W as in decode_mfma_item: 1 = the wave walks its partition, > 1 = W waves of the workgroup share it.
template <typename T, int NCH, int W, int D>
__device__ __forceinline__ void decode_mfma_int8_item(const DecodeArgs& a, int b, int p, int slice, int w) {
  static_assert(NCH == 1, "one chunk of up to 16 heads");
  static_assert(D == 128 || D == 64, "one or two 64-dim steps");
  constexpr int kSteps = D / 64;               // 64-dim steps of the first product
  const bool owns = D == 128 || (threadIdx.x & 15) < D / 8;   // this lane's 8 output dims exist
  const int lane = threadIdx.x & 63;
  const HeadSlice hs = head_slice(a, slice);
  const int g = hs.kvh;                // kv head
  const int group = hs.heads;          // q heads of this wave (<= 16)
  const int q4 = lane >> 4;            // token class: tokens 4*q4 .. 4*q4+3 of a tile
  const int col = lane & 15;           // head (first product), dim group (second product)
  const int bs = a.block_size;
  const int part_start = p * a.part_tokens;
  const int first = part_start + (W == 1 ? 0 : w * kTile);      // first token of this wave's first tile
  const int32_t* table = a.block_tables + (int64_t)b * a.max_num_blocks;
  int bi = first / bs;
  int off = first - bi * bs;
  int win_base = bi;
  int win;
  if constexpr (W > 1) win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;   // before the context length

  const int ctx = (int)load_ctx(a, b);
  // a sequence that fits one partition (or is empty) is finished here: partition 0 writes the output row
  const bool direct = ctx <= a.part_tokens;
  if (part_start >= ctx && !(direct && p == 0)) return;
  const int part_end = min(ctx, part_start + a.part_tokens);
  const int tiles_all = part_end > part_start ? (part_end - part_start + kTile - 1) / kTile : 0;
  const int ntiles = W == 1 ? tiles_all : (tiles_all > w ? (tiles_all - w + W - 1) / W : 0);   // this wave's
  if constexpr (W == 1) win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;

  // ---- query -> int8 hi/lo planes (B operand: column lane%16 -> head, bytes 16*q4.. of each 64-dim step)
  v4i qhi[kSteps], qlo[kSteps];
  float qscale;                        // amax/16256 * scale*log2e of this lane's head
  {
    const T* q = reinterpret_cast<const T*>(a.q);
    const bool live = col < group;
    const T* src = q + ((int64_t)b * a.num_heads + hs.head0 + (live ? col : 0)) * D;
    float x[kSteps][16];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < kSteps; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        x[j][e] = live ? to_float(src[64 * j + 16 * q4 + e]) : 0.f;
        amax = fmaxf(amax, fabsf(x[j][e]));
      }
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
    const float to_fix = amax > 0.f ? 16256.f / amax : 0.f;
    qscale = amax * (1.f / 16256.f) * a.scale_log2;
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      int hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int q16 = (int)rintf(x[j][e] * to_fix);            // |q16| <= 16256
        const int l8 = ((q16 + 64) & 127) - 64;                  // [-64, 63]
        const int h8 = (q16 - l8) >> 7;                          // [-127, 127]
        hi[e >> 2] |= (h8 & 0xff) << (8 * (e & 3));
        lo[e >> 2] |= (l8 & 0xff) << (8 * (e & 3));
      }
      qhi[j] = (v4i){hi[0], hi[1], hi[2], hi[3]};
      qlo[j] = (v4i){lo[0], lo[1], lo[2], lo[3]};
    }
  }

  float m = -INFINITY;      // running maximum of score + log2 v_scale of head `col`, the same in its four lanes
  float l = 0.f;            // this lane's share of the denominator (its four tokens)
  float wsum = 0.f;         // this lane's share of the sum of weights as the second product uses them
  v4f o[8];                 // o[e][j] = O[head 4*q4 + j][dim 8*col + e] (+ the bias)
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (v4f){0.f, 0.f, 0.f, 0.f};

  const int64_t row = (int64_t)a.num_kv_heads * D;          // bytes per token row
  const char* kc = reinterpret_cast<const char*>(a.k_cache) + (int64_t)g * D;
  const char* vc = reinterpret_cast<const char*>(a.v_cache) + (int64_t)g * D;
  const int k_lane_off = col * (int)row + q4 * 16;          // token lane%16, bytes 16*q4 (+64 j)
  const int v_lane_off = 4 * q4 * (int)row + col * 8;       // tokens 4*q4 + i, dims 8*(lane%16)
  const int s_lane_tok = 4 * q4 + (lane & 3);               // token whose scales this lane loads

  auto load_tile = [&](KVTileI8& t, int tile) {
    t.t0 = first + tile * (W * kTile);
    if (bi - win_base >= 64) {
      win_base = bi;
      win = (win_base + lane < a.max_num_blocks) ? table[win_base + lane] : -1;
    }
    const int phys = __builtin_amdgcn_readlane(win, bi - win_base);
    t.ok = (bi < a.max_num_blocks) && phys >= 0 && (int64_t)phys < a.num_blocks;
    if (t.ok) {
      const int64_t tok0 = (int64_t)phys * bs + off;
      const char* kp = kc + tok0 * row + k_lane_off;
      const char* vp = vc + tok0 * row + v_lane_off;
#pragma unroll
      for (int j = 0; j < kSteps; ++j) t.k[j] = *reinterpret_cast<const uint4*>(kp + 64 * j);
#pragma unroll
      for (int i = 0; i < 4; ++i) t.v[i] = owns ? load8_stream(vp + i * row) : make_uint2(0u, 0u);
      const int64_t sidx = (tok0 + s_lane_tok) * a.num_kv_heads + g;
      t.ks = a.k_scale[sidx];
      t.vs = a.v_scale[sidx];
    } else {
#pragma unroll
      for (int j = 0; j < kSteps; ++j) t.k[j] = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
      for (int i = 0; i < 4; ++i) t.v[i] = make_uint2(0u, 0u);
      t.ks = t.vs = 0.f;
    }
    if constexpr (W == 1) {
      off += kTile;
      if (off >= bs) { off = 0; ++bi; }
    } else {
      off += W * kTile;
      while (off >= bs) { off -= bs; ++bi; }
    }
  };

  auto consume = [&](const KVTileI8& t) {
    if constexpr (MVLLM_DECODE_LOADS_ONLY) {
      uint32_t x = __float_as_uint(t.ks) ^ __float_as_uint(t.vs);
#pragma unroll
      for (int j = 0; j < kSteps; ++j) x ^= t.k[j].x ^ t.k[j].y ^ t.k[j].z ^ t.k[j].w;
#pragma unroll
      for (int i = 0; i < 4; ++i) x ^= t.v[i].x ^ t.v[i].y;
      l += __uint_as_float(x & 1u);
      return;
    }
    const int tok_base = t.t0 + 4 * q4;
    const bool partial = (!t.ok) || (t.t0 + kTile > part_end);
    const float ks4[4] = {quad_bcast<0>(t.ks), quad_bcast<1>(t.ks), quad_bcast<2>(t.ks), quad_bcast<3>(t.ks)};
    float vs4[4] = {quad_bcast<0>(t.vs), quad_bcast<1>(t.vs), quad_bcast<2>(t.vs), quad_bcast<3>(t.vs)};
    if (partial) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (!t.ok || tok_base + r >= part_end) vs4[r] = 0.f;     // stale scale memory must not meet p = 0
    }
    // log2 of the V scales: the weight of a token in the second product is p * v_scale = exp2(score + log2
    // v_scale - m), and m tracks the maximum of score + log2 v_scale, so that weights stay in (0, 2^8] whatever
    // the scales are and fit fp16 (a zero scale counts as 2^-40: such a token has only zero codes)
    float lv4[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) lv4[r] = __log2f(fmaxf(vs4[r], 9.094947e-13f));
    v4i shi = {0, 0, 0, 0}, slo = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      const v4i kf = (v4i){(int)t.k[j].x, (int)t.k[j].y, (int)t.k[j].z, (int)t.k[j].w};
      shi = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf, qhi[j], shi, 0, 0, 0);
      slo = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf, qlo[j], slo, 0, 0, 0);
    }
    float s2[4], t2[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s2[r] = (float)(shi[r] * 128 + slo[r]) * (qscale * ks4[r]);
      if (partial && (!t.ok || tok_base + r >= part_end)) s2[r] = -INFINITY;
      t2[r] = s2[r] + lv4[r];
    }
    const float tile_max = fmaxf(fmaxf(t2[0], t2[1]), fmaxf(t2[2], t2[3]));
    const bool grow = tile_max > m + kLazyRescale || (m == -INFINITY && tile_max > -INFINITY);
    if (__any(grow)) {
      // the head's maximum over its four token classes, then one decision for all four lanes
      float mh = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
      mh = fmaxf(mh, __shfl_xor(mh, 32, 64));
      const bool grow_h = mh > m + kLazyRescale || (m == -INFINITY && mh > -INFINITY);
      const float m_new = grow_h ? mh : m;
      const float al = (m_new == m) ? 1.f : safe_exp2_diff(m, m_new);
      l *= al;
      wsum *= al;
      m = m_new;
      // accumulator row j is head 4*q4 + j, whose factor sits in lane 4*q4 + j (any class would do)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float aj = __shfl(al, 4 * q4 + j, 64);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e][j] *= aj;
      }
    }
    const float m_eff = (m == -INFINITY) ? 0.f : m;
    float wr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      l += fast_exp2(s2[r] - m_eff);          // softmax denominator, in the same units as the weights / v_scale
      wr[r] = fast_exp2(t2[r] - m_eff);
    }
    const v2f16 w01 = __builtin_convertvector((v2f){wr[0], wr[1]}, v2f16);
    const v2f16 w23 = __builtin_convertvector((v2f){wr[2], wr[3]}, v2f16);
    wsum += ((float)w01[0] + (float)w01[1]) + ((float)w23[0] + (float)w23[1]);      // of the weights as they are used
    const uint2 pa = make_uint2(__builtin_bit_cast(uint32_t, w01), __builtin_bit_cast(uint32_t, w23));
    // V codes biased to 0..255; the byte of dim e of tokens (0, 1) and of tokens (2, 3) as fp16 pairs 1024 + u.
    // Rows past the end hold arbitrary bytes, which are finite numbers here and meet a weight of zero.
    const uint32_t v0[2] = {t.v[0].x ^ 0x80808080u, t.v[0].y ^ 0x80808080u};
    const uint32_t v1[2] = {t.v[1].x ^ 0x80808080u, t.v[1].y ^ 0x80808080u};
    const uint32_t v2[2] = {t.v[2].x ^ 0x80808080u, t.v[2].y ^ 0x80808080u};
    const uint32_t v3[2] = {t.v[3].x ^ 0x80808080u, t.v[3].y ^ 0x80808080u};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t sel = 0x0c040c00u + 0x00010001u * (uint32_t)(e & 3);
      const uint2 vb = make_uint2(__builtin_amdgcn_perm(v1[e >> 2], v0[e >> 2], sel) | 0x64006400u,
                                  __builtin_amdgcn_perm(v3[e >> 2], v2[e >> 2], sel) | 0x64006400u);
      o[e] = mfma16x16x16<f16_t>(pa, vb, o[e]);
    }
  };

  // tiles in pairs, the odd one after the loop (see the 16-bit kernel)
  KVTileI8 ta, tb;
  if (ntiles > 0) load_tile(ta, 0);
  int tile = 0;
  for (; tile + 1 < ntiles; tile += 2) {
    load_tile(tb, tile + 1);
    consume(ta);
    if (tile + 2 < ntiles) load_tile(ta, tile + 2);
    consume(tb);
  }
  if (tile < ntiles) consume(ta);

  if constexpr (W > 1) {
    // waves 1 .. W-1 leave m, l, the weight sum and their accumulators in LDS, wave 0 folds them in (as in
    // DecodeHead::merge) and goes on alone
    __shared__ float4 part[(W - 1) * 9 * 64];
    if (w > 0) {
      float4* dst = part + (w - 1) * 9 * 64 + lane;
      dst[0] = make_float4(m, l, wsum, 0.f);
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[(1 + e) * 64] = make_float4(o[e][0], o[e][1], o[e][2], o[e][3]);
    }
    __syncthreads();
    if (w > 0) return;
#pragma unroll 1
    for (int x = 0; x < W - 1; ++x) {
      const float4* src = part + x * 9 * 64 + lane;
      const float4 mlw = src[0];
      const float m_new = fmaxf(m, mlw.x);
      const float f0 = safe_exp2_diff(m, m_new);
      const float f1 = safe_exp2_diff(mlw.x, m_new);
      m = m_new;
      l = l * f0 + mlw.y * f1;
      wsum = wsum * f0 + mlw.z * f1;
      float a0[4], a1[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        a0[j] = __shfl(f0, 4 * q4 + j, 64);
        a1[j] = __shfl(f1, 4 * q4 + j, 64);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float4 ow = src[(1 + e) * 64];
        o[e][0] = o[e][0] * a0[0] + ow.x * a1[0];
        o[e][1] = o[e][1] * a0[1] + ow.y * a1[1];
        o[e][2] = o[e][2] * a0[2] + ow.z * a1[2];
        o[e][3] = o[e][3] * a0[3] + ow.w * a1[3];
      }
    }
  }

  // denominators and weight sums over the four token classes (every lane of a head then holds the head's totals)
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  wsum += __shfl_xor(wsum, 16, 64);
  wsum += __shfl_xor(wsum, 32, 64);
  const int head0 = hs.head0;
  const float linv = l > 0.f ? 1.f / l : 0.f;
  const int64_t slot = ((int64_t)b * a.num_parts + p) * a.num_heads + head0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int h = 4 * q4 + j;
    const float bias = 1152.f * __shfl(wsum, h, 64);          // lane h (class 0) holds head h
    const float lj = __shfl(linv, h, 64);
    if (h < group && owns) {
      if (direct) {
        T r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = from_float<T>((o[e][j] - bias) * lj);
        *reinterpret_cast<uint4*>(reinterpret_cast<T*>(a.out) + ((int64_t)b * a.num_heads + head0 + h) * D + col * 8) =
            *reinterpret_cast<const uint4*>(r);
      } else {
        float* dst = a.ws_acc + (slot + h) * D + col * 8;
        *reinterpret_cast<float4*>(dst) = make_float4(o[0][j] - bias, o[1][j] - bias, o[2][j] - bias, o[3][j] - bias);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(o[4][j] - bias, o[5][j] - bias, o[6][j] - bias, o[7][j] - bias);
      }
    }
  }
  if (!direct && lane < group && lane < 16) *reinterpret_cast<float2*>(a.ws_ml + (slot + lane) * 2) = make_float2(m, l);
}

// ---------------------------------------------------------------------------
// Kernels of the fast path: one workgroup per (partition, sequence, group of kv heads); the partition index is
// an upper bound, and a workgroup whose partition lies past its sequence's context returns at once.
// ---------------------------------------------------------------------------
template <typename T, int D, bool SUB = false>
// head_dim 256 holds twice the accumulators and tiles: one wave per SIMD with up to 512 registers
__global__ __launch_bounds__(D > 128 ? 256 : 512, D > 128 ? 1 : kDecodeWavesPerEu) void decode_mfma_kernel(const DecodeArgs a) {
  int b, p, hg;
  if (!decode_item<false>(a, b, p, hg)) return;
  decode_mfma_item<T, 1, D, SUB>(a, b, p, hg * (blockDim.x >> 6) + (threadIdx.x >> 6), 0);
}
// Small batches: one workgroup of W waves per (partition, sequence, kv head), the waves splitting the tiles.
template <typename T, int W, int D, bool SUB = false>
__global__ __launch_bounds__(64 * W, D > 128 ? 1 : kDecodeWavesPerEu) void decode_mfma_split_kernel(const DecodeArgs a) {
  // kv head fastest: the workgroups of one (sequence, partition) start together and read the same token rows
  const int g = blockIdx.x, b = blockIdx.z;
  const int p = (int)((blockIdx.y + (unsigned)b) % (unsigned)a.num_parts);
  decode_mfma_item<T, W, D, SUB>(a, b, p, g, threadIdx.x >> 6);
}
template <typename T, int NCH, int D>
__global__ __launch_bounds__(kDecodeI8Threads, kDecodeI8WavesPerEu) void decode_mfma_int8_kernel(const DecodeArgs a) {
  int b, p, hg;
  if (!decode_item<true>(a, b, p, hg)) return;
  decode_mfma_int8_item<T, NCH, 1, D>(a, b, p, hg * (blockDim.x >> 6) + (threadIdx.x >> 6), 0);
}
template <typename T, int W, int D>
__global__ __launch_bounds__(64 * W, kDecodeI8WavesPerEu) void decode_mfma_int8_split_kernel(const DecodeArgs a) {
  const int g = blockIdx.x, b = blockIdx.z;
  const int p = (int)((blockIdx.y + (unsigned)b) % (unsigned)a.num_parts);
  decode_mfma_int8_item<T, 1, W, D>(a, b, p, g, threadIdx.x >> 6);
}

// ---------------------------------------------------------------------------
// Generic path: any element type (fp32 included), head_dim <= 512, any
// block_size and group size.  One wave per (partition, sequence, q head);
// lanes split head_dim, one token per step.  Correctness path for shapes the
// MFMA kernel is not built for.
// ---------------------------------------------------------------------------
constexpr int kGenericMaxR = 8;  // head_dim <= 64 * 8

template <typename T, bool INT8>
__global__ __launch_bounds__(64) void decode_generic_kernel(const DecodeArgs a) {
  const int lane = threadIdx.x;
  const int b = blockIdx.y;
  const int p = (int)((blockIdx.x + (unsigned)b) % (unsigned)a.num_parts);   // see decode_mfma_kernel
  const int h = blockIdx.z;
  const int D = a.head_dim;
  const int group = a.num_heads / a.num_kv_heads;
  const int g = h / group;

  const int ctx = (int)load_ctx(a, b);
  // a sequence that fits one partition (or is empty) is finished here: partition 0 writes the output row
  const bool direct = ctx <= a.part_tokens;
  const int part_start = p * a.part_tokens;
  if (part_start >= ctx && !(direct && p == 0)) return;
  const int part_end = min(ctx, part_start + a.part_tokens);

  float qv[kGenericMaxR], acc[kGenericMaxR];
  const T* q = reinterpret_cast<const T*>(a.q) + ((int64_t)b * a.num_heads + h) * D;
#pragma unroll
  for (int r = 0; r < kGenericMaxR; ++r) {
    const int d = lane + 64 * r;
    qv[r] = d < D ? to_float(q[d]) : 0.f;
    acc[r] = 0.f;
  }
  float m = -INFINITY, l = 0.f;
  const int bs = a.block_size;
  const int32_t* table = a.block_tables + (int64_t)b * a.max_num_blocks;
  const int64_t row = (int64_t)a.num_kv_heads * D;

  for (int t = part_start; t < part_end; ++t) {
    const int bi = t / bs;
    if (bi >= a.max_num_blocks) break;
    const int phys = table[bi];
    if (phys < 0 || (int64_t)phys >= a.num_blocks) continue;
    const int64_t tok = (int64_t)phys * bs + (t - bi * bs);
    const int64_t base = tok * row + (int64_t)g * D;
    float kscale = 1.f, vscale = 1.f;
    if (INT8) {
      kscale = a.k_scale[tok * a.num_kv_heads + g];
      vscale = a.v_scale[tok * a.num_kv_heads + g];
    }
    float kv[kGenericMaxR], vv[kGenericMaxR];
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) {
      const int d = lane + 64 * r;
      if (d < D) {
        if (INT8) {
          kv[r] = (float)reinterpret_cast<const int8_t*>(a.k_cache)[base + d] * kscale;
          vv[r] = (float)reinterpret_cast<const int8_t*>(a.v_cache)[base + d] * vscale;
        } else {
          kv[r] = to_float(reinterpret_cast<const T*>(a.k_cache)[base + d]);
          vv[r] = to_float(reinterpret_cast<const T*>(a.v_cache)[base + d]);
        }
        dot = fmaf(qv[r], kv[r], dot);
      } else {
        vv[r] = 0.f;
      }
    }
    const float s2 = wave_sum(dot) * a.scale_log2;
    const float m_new = fmaxf(m, s2);
    const float alpha = safe_exp2_diff(m, m_new);
    const float pr = fast_exp2(s2 - m_new);
    l = l * alpha + pr;
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) acc[r] = fmaf(pr, vv[r], acc[r] * alpha);
    m = m_new;
  }

  if (direct) {
    T* out = reinterpret_cast<T*>(a.out) + ((int64_t)b * a.num_heads + h) * D;
    const float linv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) {
      const int d = lane + 64 * r;
      if (d < D) out[d] = from_float<T>(acc[r] * linv);
    }
  } else {
    const int64_t slot = ((int64_t)b * a.num_parts + p) * a.num_heads + h;
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) {
      const int d = lane + 64 * r;
      if (d < D) a.ws_acc[slot * D + d] = acc[r];
    }
    if (lane == 0) {
      a.ws_ml[slot * 2] = m;
      a.ws_ml[slot * 2 + 1] = l;
    }
  }
}

// ---------------------------------------------------------------------------
// Second pass: merge the per-partition partials of one (sequence, q head).
// ---------------------------------------------------------------------------
// One wave per (sequence, query head), four heads per block; a lane owns dims lane + 64 r.  Partitions
// are folded with a running max in one pass; the loads of successive partitions do not depend on the
// arithmetic, so the unrolled loop keeps several in flight and the kernel is one short latency chain.
template <typename T>
__global__ __launch_bounds__(256) void decode_reduce_kernel(const DecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y;
  if (h >= a.num_heads) return;
  const int D = a.head_dim;
  const int ctx = (int)load_ctx(a, b);
  int np = (ctx + a.part_tokens - 1) / a.part_tokens;
  if (np > a.num_parts) np = a.num_parts;
  if (np <= 1) return;                               // written directly by the partition-0 workgroup
  const int64_t slot0 = ((int64_t)b * a.num_parts) * a.num_heads + h;
  const int64_t stride = a.num_heads;
  float acc[kGenericMaxR];
#pragma unroll
  for (int r = 0; r < kGenericMaxR; ++r) acc[r] = 0.f;
  float mx = -INFINITY, lsum = 0.f;
#pragma unroll 4
  for (int p = 0; p < np; ++p) {
    const int64_t s = slot0 + p * stride;
    const float2 ml = *reinterpret_cast<const float2*>(a.ws_ml + s * 2);
    float part[kGenericMaxR];
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) {
      const int d = lane + 64 * r;
      part[r] = d < D ? a.ws_acc[s * D + d] : 0.f;
    }
    const float mn = fmaxf(mx, ml.x);
    const float keep = safe_exp2_diff(mx, mn);
    const float wgt = safe_exp2_diff(ml.x, mn);
    lsum = lsum * keep + ml.y * wgt;
#pragma unroll
    for (int r = 0; r < kGenericMaxR; ++r) acc[r] = acc[r] * keep + part[r] * wgt;
    mx = mn;
  }
  T* out = reinterpret_cast<T*>(a.out) + ((int64_t)b * a.num_heads + h) * D;
  const float linv = lsum > 0.f ? 1.f / lsum : 0.f;
#pragma unroll
  for (int r = 0; r < kGenericMaxR; ++r) {
    const int d = lane + 64 * r;
    if (d < D) out[d] = from_float<T>(acc[r] * linv);
  }
}

// The same merge for head dims 32, 64, 128 and 256: D / 4 lanes per head with 16-byte loads, and the partials of
// eight partitions requested before the first is merged (the loop above waits for every partition in turn; a
// sequence of config 3 has up to 16 of them).  Same arithmetic in
// the same order, so the result is the same bit for bit.
template <typename T, int D>
__global__ __launch_bounds__(256) void decode_reduce_vec_kernel(const DecodeArgs a) {
  constexpr int kLanes = D / 4;                      // lanes per head
  constexpr int kBatch = 8;                          // partitions in flight (16: no faster, the short sequences' loads double)
  const int h = blockIdx.x * (256 / kLanes) + (int)threadIdx.x / kLanes;
  const int li = (int)threadIdx.x % kLanes;
  const int b = blockIdx.y;
  if (h >= a.num_heads) return;
  const int ctx = (int)load_ctx(a, b);
  int np = (ctx + a.part_tokens - 1) / a.part_tokens;
  if (np > a.num_parts) np = a.num_parts;
  if (np <= 1) return;                               // written directly by the partition-0 workgroup
  const int64_t slot0 = ((int64_t)b * a.num_parts) * a.num_heads + h;
  const int64_t stride = a.num_heads;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float mx = -INFINITY, lsum = 0.f;
  for (int p0 = 0; p0 < np; p0 += kBatch) {
    float2 ml[kBatch];
    float4 part[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      const int64_t s = slot0 + (int64_t)min(p0 + i, np - 1) * stride;     // past the last: the last again, unused
      ml[i] = *reinterpret_cast<const float2*>(a.ws_ml + s * 2);
      part[i] = *reinterpret_cast<const float4*>(a.ws_acc + s * D + 4 * li);
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (p0 + i < np) {
        const float mn = fmaxf(mx, ml[i].x);
        const float keep = safe_exp2_diff(mx, mn);
        const float wgt = safe_exp2_diff(ml[i].x, mn);
        lsum = lsum * keep + ml[i].y * wgt;
        acc[0] = acc[0] * keep + part[i].x * wgt;
        acc[1] = acc[1] * keep + part[i].y * wgt;
        acc[2] = acc[2] * keep + part[i].z * wgt;
        acc[3] = acc[3] * keep + part[i].w * wgt;
        mx = mn;
      }
    }
  }
  const float linv = lsum > 0.f ? 1.f / lsum : 0.f;
  T o4[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) o4[r] = from_float<T>(acc[r] * linv);
  T* out = reinterpret_cast<T*>(a.out) + ((int64_t)b * a.num_heads + h) * D + 4 * li;
  if constexpr (sizeof(T) == 4) *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(o4);
  else *reinterpret_cast<uint2*>(out) = *reinterpret_cast<const uint2*>(o4);
}

template <typename T>
static void launch_decode_reduce(const DecodeArgs& a, hipStream_t stream) {
  const dim3 block(256);
  const auto grid = [&](int lanes) { return dim3((unsigned)((a.num_heads + 256 / lanes - 1) / (256 / lanes)), (unsigned)a.batch); };
  // the 16-byte loads and 8- or 16-byte stores need the output rows aligned (the workspace is checked to be)
  const bool vec = (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0;
  if (vec && a.head_dim == 128) decode_reduce_vec_kernel<T, 128><<<grid(32), block, 0, stream>>>(a);
  else if (vec && a.head_dim == 64) decode_reduce_vec_kernel<T, 64><<<grid(16), block, 0, stream>>>(a);
  else if (vec && a.head_dim == 256) decode_reduce_vec_kernel<T, 256><<<grid(64), block, 0, stream>>>(a);
  else if (vec && a.head_dim == 32) decode_reduce_vec_kernel<T, 32><<<grid(8), block, 0, stream>>>(a);
  else decode_reduce_kernel<T><<<dim3((unsigned)((a.num_heads + 3) / 4), (unsigned)a.batch), block, 0, stream>>>(a);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
static size_t workspace_bytes_for(int batch, int num_heads, int head_dim, int max_num_blocks, int block_size) {
  if (batch <= 0 || num_heads <= 0 || head_dim <= 0 || max_num_blocks <= 0 || block_size <= 0) return 0;
  const int64_t max_ctx = (int64_t)max_num_blocks * block_size;
  const int part = partition_tokens_for(max_ctx, batch);
  const int64_t np = (max_ctx + part - 1) / part;
  if (np <= 1) return 0;
  return (size_t)batch * (size_t)np * (size_t)num_heads * (size_t)(head_dim + 2) * sizeof(float);
}

// Head dims the 16-bit MFMA kernels (decode, 16-row tile prefill) have instances for beside 64 and 128: the multiples
// of 8 from 32 to 120 (a last 32-dim step that is partial loads nothing past the row's end) and 256.
static bool other_mfma_dim(int head_dim) { return head_dim == 256 || (head_dim >= 32 && head_dim < 128 && head_dim % 8 == 0 && head_dim != 64); }
template <typename F>
static void with_other_mfma_dim(int head_dim, F&& go) {
  switch (head_dim) {
    case 32: go(std::integral_constant<int, 32>{}); break;
    case 40: go(std::integral_constant<int, 40>{}); break;
    case 48: go(std::integral_constant<int, 48>{}); break;
    case 56: go(std::integral_constant<int, 56>{}); break;
    case 72: go(std::integral_constant<int, 72>{}); break;
    case 80: go(std::integral_constant<int, 80>{}); break;
    case 88: go(std::integral_constant<int, 88>{}); break;
    case 96: go(std::integral_constant<int, 96>{}); break;
    case 104: go(std::integral_constant<int, 104>{}); break;
    case 112: go(std::integral_constant<int, 112>{}); break;
    case 120: go(std::integral_constant<int, 120>{}); break;
    case 256: go(std::integral_constant<int, 256>{}); break;
    default: break;
  }
}

// shapes the MFMA kernels are built for (pointer alignment is checked by the caller)
static bool fast_shape(int num_heads, int num_kv_heads, int head_dim, int block_size, int dtype, bool int8) {
  // 16-bit caches: a multiple of 8 from 32 to 128, or 256, dims per head; fp32 and INT8 caches: 64 or 128
  const bool dim_ok = head_dim == 128 || head_dim == 64 || (dtype != MVLLM_F32 && !int8 && other_mfma_dim(head_dim));
  // blocks: whole tiles; 16-bit and fp32 caches with head_dim 128 or 64 also 1, 2, 4 or 8 tokens
  const bool blocks_ok = block_size % kTile == 0 ||
                         (kTile % block_size == 0 && !int8 && (head_dim == 128 || head_dim == 64));
  return (dtype != MVLLM_F32 || !int8) && dim_ok && blocks_ok &&
         (int64_t)num_kv_heads * head_dim * 64 < ((int64_t)1 << 31);
}

// slices of up to 16 query heads per kv head (a wave's matrix tiles have 16 columns for them)
static int head_chunks_of(int num_heads, int num_kv_heads) { return (num_heads / num_kv_heads + 15) / 16; }

struct DecodePlan {
  int part_tokens, num_parts, waves_per_head;
};
static DecodePlan plan_decode(int batch, int num_kv_heads, int max_num_blocks, int block_size, bool fast_ok, bool int8) {
  const int64_t max_ctx = (int64_t)max_num_blocks * block_size;
  const bool split = fast_ok && split_wanted(max_ctx, batch, num_kv_heads, int8);
  DecodePlan plan;
  plan.part_tokens = split ? split_partition_tokens(max_ctx, batch, num_kv_heads) : partition_tokens_for(max_ctx, batch);
  plan.num_parts = (int)((max_ctx + plan.part_tokens - 1) / plan.part_tokens);
  plan.waves_per_head = !fast_ok ? 0 : split ? kSplitWaves : 1;
  return plan;
}

template <typename T> struct IsSixteenBit { static constexpr bool value = true; };
template <> struct IsSixteenBit<float> { static constexpr bool value = false; };

template <typename T>
static int launch_decode(DecodeArgs a, bool int8, bool fast_ok, bool split, hipStream_t stream) {
  bool launched = false;
  // kv heads (waves) per workgroup of the one-wave-per-head form: as many as allowed, so that a workgroup streams
  // whole token rows; fewer when the grid would otherwise leave most CUs without a workgroup
  // (a wave's unit of work is a head slice: a kv head, or 16 of its query heads where it has more than 16)
  const int slices = a.num_kv_heads * a.head_chunks;
  int wpb = largest_divisor_le(slices, int8 ? kDecodeI8Wpb : kDecodeWpb);
  while (wpb > 1 && (int64_t)a.num_parts * a.batch * (slices / wpb) < kDecodeSmallGrid)
    wpb = largest_divisor_le(slices, wpb - 1);
  const unsigned groups = (unsigned)(slices / wpb);
  const dim3 split_grid((unsigned)slices, (unsigned)a.num_parts, (unsigned)a.batch), split_block(64 * kSplitWaves);
  const dim3 block(64 * wpb);
  if (fast_ok && !int8) {
    const dim3 grid((unsigned)a.num_parts, (unsigned)a.batch, groups);
    auto go = [&](auto DIM) {
      constexpr int D = decltype(DIM)::value;
      if (split) decode_mfma_split_kernel<T, kSplitWaves, D><<<split_grid, split_block, 0, stream>>>(a);
      else decode_mfma_kernel<T, D><<<grid, block, 0, stream>>>(a);
      launched = true;
    };
    auto go_small_blocks = [&](auto DIM) {          // blocks of 1, 2, 4 or 8 tokens (head_dim 128 or 64)
      constexpr int D = decltype(DIM)::value;
      if (split) decode_mfma_split_kernel<T, kSplitWaves, D, true><<<split_grid, split_block, 0, stream>>>(a);
      else decode_mfma_kernel<T, D, true><<<grid, block, 0, stream>>>(a);
      launched = true;
    };
    if (a.block_size < kTile) {
      if (a.head_dim == 128) go_small_blocks(std::integral_constant<int, 128>{});
      else if (a.head_dim == 64) go_small_blocks(std::integral_constant<int, 64>{});
    } else {
      if (a.head_dim == 128) go(std::integral_constant<int, 128>{});
      else if (a.head_dim == 64) go(std::integral_constant<int, 64>{});
      if constexpr (IsSixteenBit<T>::value) with_other_mfma_dim(a.head_dim, go);    // 16-bit caches only
    }
  }
  if constexpr (IsSixteenBit<T>::value) {           // the INT8 kernels take 16-bit queries
    if (fast_ok && int8) {
      const dim3 grid((unsigned)a.num_parts, groups, (unsigned)a.batch);
      if (split && a.head_dim == 64) decode_mfma_int8_split_kernel<T, kSplitWaves, 64><<<split_grid, split_block, 0, stream>>>(a);
      else if (split) decode_mfma_int8_split_kernel<T, kSplitWaves, 128><<<split_grid, split_block, 0, stream>>>(a);
      else if (a.head_dim == 64) decode_mfma_int8_kernel<T, 1, 64><<<grid, block, 0, stream>>>(a);
      else decode_mfma_int8_kernel<T, 1, 128><<<grid, block, 0, stream>>>(a);
      launched = true;
    }
  }
  if (!launched) {
    dim3 grid((unsigned)a.num_parts, (unsigned)a.batch, (unsigned)a.num_heads);
    if (int8) decode_generic_kernel<T, true><<<grid, dim3(64), 0, stream>>>(a);
    else decode_generic_kernel<T, false><<<grid, dim3(64), 0, stream>>>(a);
  }
  int st = launch_status();
  if (st != 0) return st;
  if (a.num_parts > 1) {
    launch_decode_reduce<T>(a, stream);
    st = launch_status();
  }
  return st;
}

// Argument checks of the decode entry points (host only; nothing touches the device).
static int decode_check(const void* out, const void* q, const void* k_cache, const void* v_cache, const float* k_scale,
                        const float* v_scale, bool int8, const int32_t* block_tables, int max_num_blocks,
                        const void* context_lens, int batch, int num_heads, int num_kv_heads, int head_dim,
                        int block_size, int64_t num_blocks, int dtype) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
      max_num_blocks <= 0 || num_blocks < 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return MVLLM_ERR_BAD_SHAPE;
  if (batch == 0) return MVLLM_OK;
  if (!out || !q || !k_cache || !v_cache || !block_tables || !context_lens) return MVLLM_ERR_NULL_POINTER;
  if (int8 && (!k_scale || !v_scale)) return MVLLM_ERR_NULL_POINTER;
  if (head_dim > 64 * kGenericMaxR) return MVLLM_ERR_UNSUPPORTED;
  if ((int64_t)max_num_blocks * block_size > (int64_t)1 << 30) return MVLLM_ERR_UNSUPPORTED;
  if (batch > 65535 || num_heads > 65535) return MVLLM_ERR_UNSUPPORTED;
  return MVLLM_OK;
}

static int decode_entry(void* out, const void* q, const void* k_cache, const void* v_cache,
                        const float* k_scale, const float* v_scale, bool int8,
                        const int32_t* block_tables, int max_num_blocks, const void* context_lens,
                        int ctx_is_i64, int batch, int num_heads, int num_kv_heads, int head_dim,
                        int block_size, int64_t num_blocks, float scale, int dtype, void* workspace,
                        size_t workspace_bytes, void* stream) {
  const int bad = decode_check(out, q, k_cache, v_cache, k_scale, v_scale, int8, block_tables, max_num_blocks,
                               context_lens, batch, num_heads, num_kv_heads, head_dim, block_size, num_blocks, dtype);
  if (bad != MVLLM_OK) return bad;
  if (batch == 0) return MVLLM_OK;

  DecodeArgs a;
  a.out = out; a.q = q; a.k_cache = k_cache; a.v_cache = v_cache;
  a.k_scale = k_scale; a.v_scale = v_scale;
  a.block_tables = block_tables; a.context_lens = context_lens;
  a.num_blocks = num_blocks; a.ctx_is_i64 = ctx_is_i64; a.max_num_blocks = max_num_blocks;
  a.batch = batch; a.num_heads = num_heads; a.num_kv_heads = num_kv_heads; a.head_dim = head_dim;
  a.block_size = block_size;
  const bool fast_ok = fast_shape(num_heads, num_kv_heads, head_dim, block_size, dtype, int8) &&
                       aligned16(q) && aligned16(out) && aligned16(k_cache) && aligned16(v_cache);
  a.head_chunks = head_chunks_of(num_heads, num_kv_heads);
  const DecodePlan plan = plan_decode(batch, num_kv_heads * a.head_chunks, max_num_blocks, block_size, fast_ok, int8);
  const bool split = plan.waves_per_head > 1;
  a.part_tokens = plan.part_tokens;
  a.num_parts = plan.num_parts;
  a.scale_log2 = scale * kLog2e;
  a.ws_acc = nullptr; a.ws_ml = nullptr;
  if (a.num_parts > 1) {
    const size_t need = workspace_bytes_for(batch, num_heads, head_dim, max_num_blocks, block_size);
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) return MVLLM_ERR_WORKSPACE;
    a.ws_acc = reinterpret_cast<float*>(workspace);
    a.ws_ml = a.ws_acc + (size_t)batch * a.num_parts * num_heads * head_dim;
  }
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MVLLM_F32: return launch_decode<float>(a, int8, fast_ok, split, s);
    case MVLLM_BF16: return launch_decode<bf16_t>(a, int8, fast_ok, split, s);
    default: return launch_decode<f16_t>(a, int8, fast_ok, split, s);
  }
}

template <typename T, int D>
static void launch_rows16(const PrefillRowsArgs& a, dim3 grid, int tiles, hipStream_t stream) {
  if constexpr (sizeof(T) == 2 && (D == 64 || D == 128)) {
    if (a.k_scale) {
      prefill_rows16_kernel<T, D, true, true><<<grid, dim3(256), 0, stream>>>(a, tiles);
      return;
    }
  }
  if (a.block_tables) prefill_rows16_kernel<T, D, true><<<grid, dim3(256), 0, stream>>>(a, tiles);
  else prefill_rows16_kernel<T, D, false><<<grid, dim3(256), 0, stream>>>(a, tiles);
}
bool prefill_rows16_takes(int head_dim, int dtype, bool int8_cache) {
  if (head_dim == 64 || head_dim == 128) return true;
  return other_mfma_dim(head_dim) && dtype != MVLLM_F32 && !int8_cache;
}
int launch_prefill_rows16(const PrefillRowsArgs& a, int head_dim, int dtype, hipStream_t stream) {
  if (!prefill_rows16_takes(head_dim, dtype, a.k_scale != nullptr)) return MVLLM_ERR_UNSUPPORTED;
  if (a.block_tables && a.block_size % kTile != 0) return MVLLM_ERR_UNSUPPORTED;
  if (a.k_scale && (!a.v_scale || !a.block_tables || dtype == MVLLM_F32)) return MVLLM_ERR_UNSUPPORTED;
  const int64_t tiles = a.total_tokens / kTile + a.num_seqs;      // upper bound on the 16-row tiles
  const dim3 grid((unsigned)tiles, (unsigned)((a.num_heads + 3) / 4));
  if (dtype == MVLLM_F32) {
    if (head_dim == 64) launch_rows16<float, 64>(a, grid, (int)tiles, stream);
    else launch_rows16<float, 128>(a, grid, (int)tiles, stream);
  } else {
    auto go = [&](auto DIM) {
      constexpr int D = decltype(DIM)::value;
      if (dtype == MVLLM_BF16) launch_rows16<bf16_t, D>(a, grid, (int)tiles, stream);
      else launch_rows16<f16_t, D>(a, grid, (int)tiles, stream);
    };
    if (head_dim == 64) go(std::integral_constant<int, 64>{});
    else if (head_dim == 128) go(std::integral_constant<int, 128>{});
    else with_other_mfma_dim(head_dim, go);
  }
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

extern "C" size_t mvllm_paged_decode_workspace_bytes(int batch, int num_heads, int head_dim,
                                                     int max_num_blocks, int block_size) {
  return workspace_bytes_for(batch, num_heads, head_dim, max_num_blocks, block_size);
}

extern "C" int mvllm_paged_decode_plan(int batch, int num_heads, int num_kv_heads, int head_dim, int max_num_blocks,
                                       int block_size, int dtype, int int8_cache, int* part_tokens, int* num_parts,
                                       int* waves_per_head) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (batch <= 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 || max_num_blocks <= 0 ||
      num_heads % num_kv_heads != 0)
    return MVLLM_ERR_BAD_SHAPE;
  const DecodePlan plan = plan_decode(batch, num_kv_heads * head_chunks_of(num_heads, num_kv_heads), max_num_blocks, block_size,
                                      fast_shape(num_heads, num_kv_heads, head_dim, block_size, dtype, int8_cache != 0), int8_cache != 0);
  if (part_tokens) *part_tokens = plan.part_tokens;
  if (num_parts) *num_parts = plan.num_parts;
  if (waves_per_head) *waves_per_head = plan.waves_per_head;
  return MVLLM_OK;
}

extern "C" int mvllm_paged_decode(void* out, const void* q, const void* k_cache, const void* v_cache,
                                  const int32_t* block_tables, int max_num_blocks, const void* context_lens,
                                  int ctx_is_i64, int batch, int num_heads, int num_kv_heads, int head_dim,
                                  int block_size, int64_t num_blocks, float scale, int dtype, void* workspace,
                                  size_t workspace_bytes, void* stream) {
  return decode_entry(out, q, k_cache, v_cache, nullptr, nullptr, false, block_tables, max_num_blocks,
                      context_lens, ctx_is_i64, batch, num_heads, num_kv_heads, head_dim, block_size,
                      num_blocks, scale, dtype, workspace, workspace_bytes, stream);
}

// ---------------------------------------------------------------------------
// Entry point for callers that cannot allocate: the split-K partials go to a static device array instead of a
// caller-owned workspace.  The array's name is only a host-side handle; its device address is looked up once per
// device (hipGetSymbolAddress with that device current) and kept.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = MVLLM_PAGED_DECODE_NOALLOC_MAX_BYTES;   // 32 MiB per GPU
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the device that owns `stream` (the current device for the null stream): every GPU
// holds its own copy of the array at its own address, and the kernels run where the stream lives, which need not be
// the caller's current device.  Looked up once per device, with that device current for the lookup; null (and
// *status set) when it fails.
static void* static_scratch(hipStream_t stream, int* status) {
  int cur = -1;
  hipError_t e = hipGetDevice(&cur);
  if (e != hipSuccess) { *status = (int)e; return nullptr; }
  int dev = cur;
  if (stream != nullptr) {
    e = hipStreamGetDevice(stream, &dev);
    if (e != hipSuccess) { *status = (int)e; return nullptr; }
  }
  if (dev < 0 || dev >= kMaxDevices) { *status = MVLLM_ERR_UNSUPPORTED; return nullptr; }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p) return p;
  if (dev != cur && (e = hipSetDevice(dev)) != hipSuccess) { *status = (int)e; return nullptr; }
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (dev != cur) {
    const hipError_t back = hipSetDevice(cur);
    if (e == hipSuccess) e = back;
  }
  if (e != hipSuccess || !p) { *status = e != hipSuccess ? (int)e : MVLLM_ERR_WORKSPACE; return nullptr; }
  g_scratch_ptr[dev].store(p, std::memory_order_release);   // two threads racing here store the same address
  return p;
}

extern "C" int mvllm_paged_decode_noalloc(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, int max_num_blocks, const void* context_lens,
                                          int ctx_is_i64, int batch, int num_heads, int num_kv_heads, int head_dim,
                                          int block_size, int64_t num_blocks, float scale, int dtype, void* stream) {
  // arguments and sizes first, so that a bad call is refused before anything touches the device
  int status = decode_check(out, q, k_cache, v_cache, nullptr, nullptr, false, block_tables, max_num_blocks,
                            context_lens, batch, num_heads, num_kv_heads, head_dim, block_size, num_blocks, dtype);
  if (status != MVLLM_OK || batch == 0) return status;
  const size_t need = workspace_bytes_for(batch, num_heads, head_dim, max_num_blocks, block_size);
  if (need > kStaticScratchBytes) return MVLLM_ERR_WORKSPACE;
  void* ws = static_scratch((hipStream_t)stream, &status);
  if (!ws) return status;
  // Every partial a merge reads has been written by a workgroup of the same call (a sequence's live partitions
  // all run), so nothing in the array has to start at zero.
  return decode_entry(out, q, k_cache, v_cache, nullptr, nullptr, false, block_tables, max_num_blocks,
                      context_lens, ctx_is_i64, batch, num_heads, num_kv_heads, head_dim, block_size,
                      num_blocks, scale, dtype, ws, kStaticScratchBytes, stream);
}

extern "C" int mvllm_paged_decode_int8(void* out, const void* q, const int8_t* k_cache, const int8_t* v_cache,
                                       const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                       int max_num_blocks, const void* context_lens, int ctx_is_i64, int batch,
                                       int num_heads, int num_kv_heads, int head_dim, int block_size,
                                       int64_t num_blocks, float scale, int dtype, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  return decode_entry(out, q, k_cache, v_cache, k_scale, v_scale, true, block_tables, max_num_blocks,
                      context_lens, ctx_is_i64, batch, num_heads, num_kv_heads, head_dim, block_size,
                      num_blocks, scale, dtype, workspace, workspace_bytes, stream);
}
