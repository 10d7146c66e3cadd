// Prefill over a paged cache (16-bit, or INT8 codes with fp32 scales) with the keys of every sequence cut into ranges: a batch of few new tokens behind
// long cached prefixes (a follow-up turn of a chat, the last chunk of a chunked prefill) has too few query tiles to
// occupy the chip, and every one of them walks the whole prefix.  Here a sequence's prefix is cut into `splits - 1`
// ranges of whole key tiles and whole cache blocks plus one last range that holds the rest of the prefix and the new
// tokens; the one-group kernel of prefill_mfma.h walks each range as a sequence of its own (same queries, a block table
// that starts at the range's first block, every key of a prefix range visible, the last range causal) and writes a
// partial result and the logarithm of its softmax denominator per (query row, head); a second kernel merges them.
// Three launches: the plan (tables and offsets of the ranges, from lengths that only the device holds), the attention
// kernel, the merge.  No counterpart in the reference (its Triton prefill never reads the paged cache,
// attention.py:111-209).
#include <algorithm>

#include "common.h"
#include "prefill_mfma.h"

namespace mvllm {

namespace {

constexpr int kMaxRanges = 64;         // ranges of all sequences together: one wave plans them, and the attention kernel
                                       // deals the work of at most 64 sequences heaviest first

struct SplitArgs {
  const int32_t* cu_seqlens_q;
  const int32_t* cu_seqlens_k;
  const int32_t* block_tables;
  int32_t* ws_cu_q;        // [ranges + 1]
  int32_t* ws_cu_k;        // [ranges + 1]
  int32_t* ws_q_pos;       // [ranges]
  int32_t* ws_table;       // [ranges, table_width]
  int num_seqs;
  int splits;
  int unit;                // keys: a common multiple of the key tile (64) and the block size
  int block_size;
  int max_num_blocks;
  int table_width;
  int total_q;
};

struct Range { int key0, keys, q_pos; };
// Range i of sequence s (range numbering: i * num_seqs + s).
__device__ __forceinline__ Range range_of(const SplitArgs& a, int s, int i) {
  const int n = a.cu_seqlens_q[s + 1] - a.cu_seqlens_q[s];
  const int kv = a.cu_seqlens_k[s + 1] - a.cu_seqlens_k[s];
  const int cached = max(kv - n, 0);
  const int units = cached / a.unit;                           // whole units of the prefix
  const int per = (units + a.splits - 2) / (a.splits - 1);     // units per prefix range
  Range r;
  if (i < a.splits - 1) {
    const int u0 = min(i * per, units), u1 = min((i + 1) * per, units);
    r.key0 = u0 * a.unit;
    r.keys = n > 0 ? (u1 - u0) * a.unit : 0;
    r.q_pos = r.keys;                                          // every query row sees the whole range
  } else {
    r.key0 = units * a.unit;
    r.keys = n > 0 ? kv - r.key0 : 0;
    r.q_pos = cached - r.key0;
  }
  return r;
}

// Workgroup v: the block table of range v; workgroup 0 also the offsets of all ranges.
__global__ __launch_bounds__(64) void split_plan_kernel(const SplitArgs a) {
  const int ranges = a.num_seqs * a.splits;
  const int lane = threadIdx.x;
  if (blockIdx.x == 0) {
    int keys = 0;
    if (lane < ranges) {
      const int i = lane / a.num_seqs, s = lane - i * a.num_seqs;
      const Range r = range_of(a, s, i);
      keys = r.keys;
      a.ws_q_pos[lane] = r.q_pos;
      a.ws_cu_q[lane] = i * a.total_q + a.cu_seqlens_q[s];
    }
    int sum = keys;                                            // inclusive scan over the wave
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(sum, d, 64);
      if (lane >= d) sum += up;
    }
    if (lane < ranges) a.ws_cu_k[lane + 1] = sum;
    if (lane == 0) {
      a.ws_cu_k[0] = 0;
      a.ws_cu_q[ranges] = a.splits * a.total_q;
    }
  }
  const int v = blockIdx.x;
  const int i = v / a.num_seqs, s = v - i * a.num_seqs;
  const Range r = range_of(a, s, i);
  const int b0 = r.key0 / a.block_size;
  const int nb = (r.keys + a.block_size - 1) / a.block_size;
  const int32_t* src = a.block_tables + (int64_t)s * a.max_num_blocks;
  int32_t* dst = a.ws_table + (int64_t)v * a.table_width;
  for (int b = lane; b < a.table_width; b += 64) dst[b] = b < nb && b0 + b < a.max_num_blocks ? src[b0 + b] : -1;
}

struct MergeArgs {
  void* out;               // [total_q, Hq, D]
  const void* part;        // [splits * total_q, Hq, D]
  const float* lse;        // [splits * total_q, Hq]
  const int32_t* cu_seqlens_q;
  const int32_t* ws_cu_k;
  int num_seqs;
  int splits;
  int total_q;
  int num_heads;
  int head_dim;
};

// One workgroup per (query row, slice of floor(256 / (D / 8)) heads); a thread merges 8 output elements of one head.  out =
// sum_i 2^(lse_i - M) o_i / sum_i 2^(lse_i - M) over the ranges that hold keys, M their largest lse: o_i is range i's
// normalised result and 2^lse_i its softmax denominator, so the weights restore the numerators.  The denominators of
// the slice are fetched into LDS first, all at once (an empty range's as -inf, which weighs it out), so that the loop
// over the ranges has nothing to wait for but its own independent loads.
template <typename T>
__global__ __launch_bounds__(256) void split_merge_kernel(const MergeArgs a) {
  __shared__ float lse_s[kMaxRanges][64];
  const int t = blockIdx.x;
  const int chunks = a.head_dim / 8;               // 4 .. 32
  const int heads_here = 256 / chunks;             // 64 .. 8
  const int head0 = blockIdx.y * heads_here;
  int s = 0;
  while (s + 1 < a.num_seqs && a.cu_seqlens_q[s + 1] <= t) ++s;
  for (int idx = threadIdx.x; idx < a.splits * heads_here; idx += 256) {
    const int i = idx / heads_here, hh = idx - i * heads_here;
    const int v = i * a.num_seqs + s;
    float x = -INFINITY;
    if (head0 + hh < a.num_heads && a.ws_cu_k[v + 1] - a.ws_cu_k[v] > 0)
      x = a.lse[((int64_t)i * a.total_q + t) * a.num_heads + head0 + hh];
    lse_s[i][hh] = x;
  }
  __syncthreads();
  const int hh = threadIdx.x / chunks, c = threadIdx.x - hh * chunks;
  const int h = head0 + hh;
  if (hh >= heads_here || h >= a.num_heads) return;
  float top = -INFINITY;
  for (int i = 0; i < a.splits; ++i) top = fmaxf(top, lse_s[i][hh]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  const T* part = reinterpret_cast<const T*>(a.part) + ((int64_t)t * a.num_heads + h) * a.head_dim + 8 * c;
  const int64_t stride = (int64_t)a.total_q * a.num_heads * a.head_dim;     // one range's partial results
#pragma unroll 4
  for (int i = 0; i < a.splits; ++i) {
    const float x = lse_s[i][hh];
    const float w = x == -INFINITY ? 0.f : exp2f(x - top);
    // an empty range's rows were never written: read them (the memory is the workspace's) but weigh them by a select,
    // not a product, so that whatever bits they hold stay out
    const uint4 p = *reinterpret_cast<const uint4*>(part + i * stride);
    den += w;
    const uint32_t words[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[2 * e] = w != 0.f ? fmaf(w, lo_to_float<T>(words[e]), acc[2 * e]) : acc[2 * e];
      acc[2 * e + 1] = w != 0.f ? fmaf(w, hi_to_float<T>(words[e]), acc[2 * e + 1]) : acc[2 * e + 1];
    }
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
  uint4 o;
  o.x = pack2<T>(acc[0] * inv, acc[1] * inv);
  o.y = pack2<T>(acc[2] * inv, acc[3] * inv);
  o.z = pack2<T>(acc[4] * inv, acc[5] * inv);
  o.w = pack2<T>(acc[6] * inv, acc[7] * inv);
  *reinterpret_cast<uint4*>(reinterpret_cast<T*>(a.out) + ((int64_t)t * a.num_heads + h) * a.head_dim + 8 * c) = o;
}

int gcd_int(int x, int y) {
  while (y != 0) {
    const int r = x % y;
    x = y;
    y = r;
  }
  return x;
}

struct SplitLayout {
  int unit;
  int table_width;
  size_t ints_bytes;       // offsets, positions and tables, rounded up to 256
  size_t part_bytes;       // partial results, rounded up to 256
  size_t total_bytes;
};
SplitLayout split_layout(int num_seqs, int64_t total_q, int max_kv_len, int num_heads, int head_dim, int block_size, int splits) {
  SplitLayout l;
  l.unit = block_size / gcd_int(block_size, 64) * 64;
  const int ranges = num_seqs * splits;
  const int64_t units = max_kv_len / l.unit;
  const int64_t per = (units + splits - 2) / (splits - 1);
  const int64_t prefix_keys = per * l.unit;                                  // longest prefix range
  const int64_t last_keys = std::min<int64_t>(max_kv_len, l.unit + total_q); // longest last range
  l.table_width = (int)((std::max(prefix_keys, last_keys) + block_size - 1) / block_size) + 1;
  const size_t ints = (size_t)(2 * (ranges + 1) + ranges) + (size_t)ranges * l.table_width;
  l.ints_bytes = (ints * sizeof(int32_t) + 255) / 256 * 256;
  l.part_bytes = ((size_t)splits * total_q * num_heads * head_dim * 2 + 255) / 256 * 256;
  const size_t lse_bytes = ((size_t)splits * total_q * num_heads * sizeof(float) + 255) / 256 * 256;
  l.total_bytes = l.ints_bytes + l.part_bytes + lse_bytes;
  return l;
}

// int8: an INT8 cache (head_dim 64 and 128 only; a 16-bit cache also the other head dims of the LDS-tiled kernel)
bool split_shape_ok(int num_seqs, int64_t total_q, int max_kv_len, int num_heads, int num_kv_heads, int head_dim,
                    int block_size, int dtype, int splits, bool int8) {
  if (num_seqs <= 0 || total_q <= 0 || max_kv_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || block_size <= 0) return false;
  if (num_heads % num_kv_heads != 0 || num_heads > 65535) return false;
  if (dtype != MVLLM_BF16 && dtype != MVLLM_F16) return false;
  const bool dim_ok = head_dim == 128 || head_dim == 64 || (!int8 && prefill_mfma_other_dim(head_dim));
  if (!dim_ok || block_size % 16 != 0 || block_size > (1 << 20)) return false;
  if ((int64_t)block_size * num_kv_heads * head_dim * (int8 ? 1 : 2) >= ((int64_t)1 << 31)) return false;
  if (splits < 2 || (int64_t)num_seqs * splits > kMaxRanges) return false;
  if ((int64_t)splits * total_q > ((int64_t)1 << 30)) return false;
  return true;
}

}  // namespace

}  // namespace mvllm

using namespace mvllm;

// How many ranges to cut every sequence's keys into for a batch of these sizes (total_q_tokens new tokens in num_seqs
// sequences, the longest of max_kv_len keys): 0 = do not split (enough query tiles to fill the chip, keys too few to be
// worth the two extra launches, or a shape the split form is not built for).  The numbers: the two-group kernel deals
// items of 64 rows x 4 heads to 256 compute units, and a launch of fewer than 192 of them leaves a quarter of the chip
// idle from the start (shapes it does not take: fewer than three quarters of the one-group kernel's 512 places, 256 at head_dim 256);
// the one-group kernel that walks the ranges runs two workgroups per compute unit, so the ranges
// aim at 512 workgroups in all (but at 4 prefix ranges at least), each prefix range at least 1024 keys long, at most 16
// of them (more only lengthen the merge).
extern "C" int mvllm_prefill_paged_split_plan(int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                              int num_kv_heads, int head_dim, int block_size, int dtype, int int8_cache) {
  if (!split_shape_ok(num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, dtype, 2, int8_cache != 0))
    return 0;
  if (max_kv_len < 4096) return 0;
  const int group = num_heads / num_kv_heads;
  const int hpw = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
  const int rows = 32 * (4 / hpw);                    // query rows of a one-group workgroup
  // one-group workgroups of one range (every sequence but one may add a partial row tile)
  const int64_t items = ((total_q_tokens + rows - 1) / rows + num_seqs - 1) * (num_heads / hpw);
  const int places = head_dim == 256 ? 256 : 512;     // workgroups of the one-group kernel the chip holds at a time
  // what the call would run on otherwise: the two-group kernel (for an INT8 cache behind the staging step), or the
  // one-group kernel with its 512 places
  if (prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, 16)) {
    const int64_t wide_items = (total_q_tokens / 64 + num_seqs) * std::max(num_heads / 4, 1);
    // INT8: the ranges run on the one-step kernel, which converts every tile for every query tile (two thirds of the
    // two-step form's rate), so the chip has to be emptier for the cut to pay (2 x 512 tokens behind 16384: 362 us in
    // two steps, 406 us cut)
    if (wide_items >= (int8_cache != 0 ? 96 : 192)) return 0;
  } else if (items >= 3 * places / 4) {
    return 0;
  }
  int64_t prefix_ranges = std::max<int64_t>(places / items - 1, 4);   // 4: a batch this small gains from any cut (measured)
  prefix_ranges = std::min<int64_t>(prefix_ranges, max_kv_len / 1024);
  prefix_ranges = std::min<int64_t>(prefix_ranges, kMaxRanges / num_seqs - 1);
  prefix_ranges = std::min<int64_t>(prefix_ranges, 16);
  return prefix_ranges >= 2 ? (int)prefix_ranges + 1 : 0;
}

extern "C" size_t mvllm_prefill_paged_split_workspace_bytes(int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                                            int num_kv_heads, int head_dim, int block_size, int dtype, int splits) {
  if (!split_shape_ok(num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, dtype, splits, false)) return 0;
  return split_layout(num_seqs, total_q_tokens, max_kv_len, num_heads, head_dim, block_size, splits).total_bytes;
}

static int run_split(void* out, const void* q, const void* k_cache, const void* v_cache, const float* k_scale,
                     const float* v_scale, bool int8, const int32_t* block_tables, int max_num_blocks,
                     const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int num_seqs, int64_t total_q_tokens,
                     int max_kv_len, int num_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                     float scale, int dtype, int splits, void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_q_tokens < 0 || max_kv_len < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 ||
      block_size <= 0 || num_blocks < 0 || max_num_blocks < 0 || num_heads % num_kv_heads != 0 || !(scale > 0.f))
    return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_q_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k_cache || !v_cache || (int8 && (!k_scale || !v_scale)) || !block_tables || !cu_seqlens_q || !cu_seqlens_k)
    return MVLLM_ERR_NULL_POINTER;
  if (!split_shape_ok(num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, dtype, splits, int8))
    return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(out) || !aligned16(k_cache) || !aligned16(v_cache)) return MVLLM_ERR_MISALIGNED;
  const SplitLayout l = split_layout(num_seqs, total_q_tokens, max_kv_len, num_heads, head_dim, block_size, splits);
  if (!workspace || workspace_bytes < l.total_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return MVLLM_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  const int ranges = num_seqs * splits;
  int32_t* ints = reinterpret_cast<int32_t*>(workspace);
  SplitArgs sp;
  sp.cu_seqlens_q = cu_seqlens_q; sp.cu_seqlens_k = cu_seqlens_k; sp.block_tables = block_tables;
  sp.ws_cu_q = ints;
  sp.ws_cu_k = ints + (ranges + 1);
  sp.ws_q_pos = ints + 2 * (ranges + 1);
  sp.ws_table = ints + 2 * (ranges + 1) + ranges;
  sp.num_seqs = num_seqs; sp.splits = splits; sp.unit = l.unit; sp.block_size = block_size;
  sp.max_num_blocks = max_num_blocks; sp.table_width = l.table_width; sp.total_q = (int)total_q_tokens;
  split_plan_kernel<<<dim3((unsigned)ranges), dim3(64), 0, s>>>(sp);
  int status = launch_status();
  if (status != MVLLM_OK) return status;

  char* part = reinterpret_cast<char*>(workspace) + l.ints_bytes;
  float* lse = reinterpret_cast<float*>(part + l.part_bytes);
  PrefillArgs a;
  a.out = part; a.q = q; a.k = k_cache; a.v = v_cache; a.cu_seqlens = sp.ws_cu_q;
  a.total_tokens = (int64_t)splits * total_q_tokens; a.num_seqs = ranges; a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
  a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
  a.cu_seqlens_k = sp.ws_cu_k; a.block_tables = sp.ws_table; a.max_num_blocks = l.table_width;
  a.block_size = block_size; a.num_blocks = num_blocks; a.k_scale = k_scale; a.v_scale = v_scale;
  a.q_pos = sp.ws_q_pos; a.lse = lse; a.q_period = total_q_tokens;
  status = int8                               ? launch_prefill_paged_int8(a, dtype, s)
           : prefill_mfma_other_dim(head_dim) ? launch_prefill_mfma_other(a, dtype, true, s)
                                              : launch_prefill_paged_16bit(a, dtype, s);
  if (status != MVLLM_OK) return status;

  MergeArgs m;
  m.out = out; m.part = part; m.lse = lse; m.cu_seqlens_q = cu_seqlens_q; m.ws_cu_k = sp.ws_cu_k;
  m.num_seqs = num_seqs; m.splits = splits; m.total_q = (int)total_q_tokens; m.num_heads = num_heads; m.head_dim = head_dim;
  const int heads_per_wg = 256 / (head_dim / 8);
  const dim3 grid((unsigned)total_q_tokens, (unsigned)((num_heads + heads_per_wg - 1) / heads_per_wg));
  if (dtype == MVLLM_BF16) split_merge_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(m);
  else split_merge_kernel<f16_t><<<grid, dim3(256), 0, s>>>(m);
  return launch_status();
}

extern "C" int mvllm_prefill_paged_split(void* out, const void* q, const void* k_cache, const void* v_cache,
                                         const int32_t* block_tables, int max_num_blocks, const int32_t* cu_seqlens_q,
                                         const int32_t* cu_seqlens_k, int num_seqs, int64_t total_q_tokens, int max_kv_len,
                                         int num_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                                         float scale, int dtype, int splits, void* workspace, size_t workspace_bytes,
                                         void* stream) {
  return run_split(out, q, k_cache, v_cache, nullptr, nullptr, false, block_tables, max_num_blocks, cu_seqlens_q, cu_seqlens_k,
                   num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, dtype,
                   splits, workspace, workspace_bytes, stream);
}

extern "C" int mvllm_prefill_paged_int8_split(void* out, const void* q, const int8_t* k_cache, const int8_t* v_cache,
                                              const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                              int max_num_blocks, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                              int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                              int num_kv_heads, int head_dim, int block_size, int64_t num_blocks, float scale,
                                              int dtype, int splits, void* workspace, size_t workspace_bytes, void* stream) {
  return run_split(out, q, k_cache, v_cache, k_scale, v_scale, true, block_tables, max_num_blocks, cu_seqlens_q, cu_seqlens_k,
                   num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, dtype,
                   splits, workspace, workspace_bytes, stream);
}
