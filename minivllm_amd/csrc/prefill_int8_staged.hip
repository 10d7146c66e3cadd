// Prefill over an INT8 paged cache in two steps: the keys and values of every sequence of the batch are dequantised
// once (code * scale, rounded to the query's 16-bit type: the values the one-step kernel of prefill_mfma.h feeds the
// matrix unit) into a caller-provided workspace laid out as a 16-bit paged cache with blocks of 16 tokens, then the
// two-group kernel of prefill_pingpong.hip (shapes it does not take: the one-group kernel's 16-bit paged form) runs over
// that cache.  The one-step kernel converts each K/V tile again for every 32-row query tile and head slice that walks
// it, which is most of its time; here a value is converted once and read back as often as the kernel needs it.  No
// counterpart in the reference (it has no INT8 cache).
#include "common.h"
#include "prefill_mfma.h"

namespace mvllm {

namespace {

constexpr int kStageBlock = 16;        // tokens per block of the staged cache

struct StageArgs {
  const int8_t* k_codes;
  const int8_t* v_codes;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_tables;
  const int32_t* cu_seqlens_k;
  void* ws_k;
  void* ws_v;
  int32_t* ws_table;
  int64_t num_blocks;
  int max_num_blocks;
  int block_size;
  int num_kv_heads;
  int head_dim;
  int blocks_per_seq;      // blocks of the staged cache per sequence
};

// One workgroup per (16-token block, sequence): its tokens' codes -> 16-bit values in the staged cache, and the
// block's entry of the staged block table.  A source block whose table entry is not a block of the pool reads as
// zeros, as in the one-step kernel.  Tokens past the sequence's last key are not written (the two-group kernel's
// copy descriptors end with the last key).
template <typename T>
__global__ __launch_bounds__(256) void stage_int8_blocks_kernel(const StageArgs a) {
  const int s = blockIdx.y, blk = blockIdx.x;
  const int staged = s * a.blocks_per_seq + blk;
  if (threadIdx.x == 0) a.ws_table[staged] = staged;
  const int kv_len = a.cu_seqlens_k[s + 1] - a.cu_seqlens_k[s];
  const int t0 = kStageBlock * blk;
  if (t0 >= kv_len) return;
  // block_size % 16 == 0: the 16 tokens lie in one source block
  const int bi = t0 / a.block_size, off0 = t0 - bi * a.block_size;
  const int phys = bi < a.max_num_blocks ? a.block_tables[(int64_t)s * a.max_num_blocks + bi] : -1;
  const bool mapped = phys >= 0 && (int64_t)phys < a.num_blocks;
  const int row_elems = a.num_kv_heads * a.head_dim;          // codes (= bytes) per token
  const int chunks = row_elems / 16;                           // 16 codes -> 32 bytes
  const int rows = kv_len - t0 < kStageBlock ? kv_len - t0 : kStageBlock;
  const int64_t src_row0 = mapped ? (int64_t)phys * a.block_size + off0 : 0;
  char* dk = reinterpret_cast<char*>(a.ws_k) + (int64_t)staged * kStageBlock * row_elems * 2;
  char* dv = reinterpret_cast<char*>(a.ws_v) + (int64_t)staged * kStageBlock * row_elems * 2;
  for (int idx = threadIdx.x; idx < rows * chunks; idx += 256) {
    const int r = idx / chunks, c = idx - r * chunks;
    uint4 k0 = make_uint4(0u, 0u, 0u, 0u), k1 = k0, v0 = k0, v1 = k0;
    if (mapped) {
      const int64_t row = src_row0 + r;
      const int kvh = 16 * c / a.head_dim;
      const float ks = a.k_scale[row * a.num_kv_heads + kvh], vs = a.v_scale[row * a.num_kv_heads + kvh];
      const uint4 ck = *reinterpret_cast<const uint4*>(a.k_codes + row * row_elems + 16 * c);
      const uint4 cv = *reinterpret_cast<const uint4*>(a.v_codes + row * row_elems + 16 * c);
      k0 = dequant8_biased<T>(ck.x, ck.y, ks, -128.f * ks);
      k1 = dequant8_biased<T>(ck.z, ck.w, ks, -128.f * ks);
      v0 = dequant8_biased<T>(cv.x, cv.y, vs, -128.f * vs);
      v1 = dequant8_biased<T>(cv.z, cv.w, vs, -128.f * vs);
    }
    uint4* ko = reinterpret_cast<uint4*>(dk + ((int64_t)r * row_elems + 16 * c) * 2);
    uint4* vo = reinterpret_cast<uint4*>(dv + ((int64_t)r * row_elems + 16 * c) * 2);
    ko[0] = k0; ko[1] = k1;
    vo[0] = v0; vo[1] = v1;
  }
}

struct StageLayout {
  int blocks_per_seq;
  size_t cache_bytes;      // one of the two staged caches
  size_t total_bytes;
};
StageLayout stage_layout(int num_seqs, int max_kv_len, int num_kv_heads, int head_dim) {
  StageLayout l;
  l.blocks_per_seq = (max_kv_len + kStageBlock - 1) / kStageBlock;
  l.cache_bytes = (size_t)num_seqs * l.blocks_per_seq * kStageBlock * num_kv_heads * head_dim * 2;
  const size_t table_bytes = ((size_t)num_seqs * l.blocks_per_seq * sizeof(int32_t) + 255) / 256 * 256;
  l.total_bytes = 2 * l.cache_bytes + table_bytes;
  return l;
}

// 2: the two-group kernel runs over the staged cache, 1: the one-group kernel, 0: this form is not built for the shape
int staged_kind(int num_seqs, int max_kv_len, int num_heads, int num_kv_heads, int head_dim, int block_size, int dtype) {
  if (num_seqs <= 0 || max_kv_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  if (block_size <= 0 || block_size % 16 != 0 || num_heads > 65535 || dtype == MVLLM_F32) return 0;
  if (head_dim != 128 && head_dim != 64) return 0;
  if ((int64_t)num_seqs * ((max_kv_len + kStageBlock - 1) / kStageBlock) >= ((int64_t)1 << 31)) return 0;
  if ((int64_t)num_kv_heads * head_dim * 64 >= ((int64_t)1 << 31)) return 0;
  return prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, kStageBlock) ? 2 : 1;
}

}  // namespace

}  // namespace mvllm

using namespace mvllm;

extern "C" size_t mvllm_prefill_paged_int8_workspace_bytes(int num_seqs, int max_kv_len, int num_heads, int num_kv_heads,
                                                           int head_dim, int block_size, int dtype) {
  if (staged_kind(num_seqs, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, dtype) == 0) return 0;
  return stage_layout(num_seqs, max_kv_len, num_kv_heads, head_dim).total_bytes;
}

extern "C" int mvllm_prefill_paged_int8_staged(void* out, const void* q, const int8_t* k_cache, const int8_t* v_cache,
                                               const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                               int max_num_blocks, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                               int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                               int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                                               float scale, int dtype, void* workspace, size_t workspace_bytes,
                                               void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_q_tokens < 0 || max_kv_len < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 ||
      block_size <= 0 || num_blocks < 0 || max_num_blocks < 0 || num_heads % num_kv_heads != 0 || !(scale > 0.f))
    return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_q_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k_cache || !v_cache || !k_scale || !v_scale || !block_tables || !cu_seqlens_q || !cu_seqlens_k)
    return MVLLM_ERR_NULL_POINTER;
  const int kind = staged_kind(num_seqs, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, dtype);
  if (total_q_tokens > ((int64_t)1 << 30) || kind == 0) return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(out) || !aligned16(k_cache) || !aligned16(v_cache)) return MVLLM_ERR_MISALIGNED;
  const StageLayout l = stage_layout(num_seqs, max_kv_len, num_kv_heads, head_dim);
  if (!workspace || workspace_bytes < l.total_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return MVLLM_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  StageArgs st;
  st.k_codes = k_cache; st.v_codes = v_cache; st.k_scale = k_scale; st.v_scale = v_scale;
  st.block_tables = block_tables; st.cu_seqlens_k = cu_seqlens_k;
  st.ws_k = workspace;
  st.ws_v = reinterpret_cast<char*>(workspace) + l.cache_bytes;
  st.ws_table = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + 2 * l.cache_bytes);
  st.num_blocks = num_blocks; st.max_num_blocks = max_num_blocks; st.block_size = block_size;
  st.num_kv_heads = num_kv_heads; st.head_dim = head_dim; st.blocks_per_seq = l.blocks_per_seq;
  const dim3 grid((unsigned)l.blocks_per_seq, (unsigned)num_seqs);
  if (dtype == MVLLM_BF16) stage_int8_blocks_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(st);
  else stage_int8_blocks_kernel<f16_t><<<grid, dim3(256), 0, s>>>(st);
  const int status = launch_status();
  if (status != MVLLM_OK) return status;
  if (kind == 1) {
    PrefillArgs a;
    a.out = out; a.q = q; a.k = st.ws_k; a.v = st.ws_v; a.cu_seqlens = cu_seqlens_q;
    a.total_tokens = total_q_tokens; a.num_seqs = num_seqs; a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
    a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
    a.cu_seqlens_k = cu_seqlens_k; a.block_tables = st.ws_table; a.max_num_blocks = l.blocks_per_seq;
    a.block_size = kStageBlock; a.num_blocks = (int64_t)num_seqs * l.blocks_per_seq; a.k_scale = nullptr; a.v_scale = nullptr;
    return launch_prefill_paged_16bit(a, dtype, s);
  }
  PrefillPpArgs p;
  p.out = out; p.q = q; p.k = st.ws_k; p.v = st.ws_v; p.cu_seqlens = cu_seqlens_q; p.total_tokens = total_q_tokens;
  p.num_seqs = num_seqs; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.scale_log2 = scale * kLog2e;
  p.slices = 0; p.n_teams = 0; p.team_size = 0; p.level_bits = 0; p.spt_magic = 0; p.chunks_magic = 0;
  p.cu_seqlens_k = cu_seqlens_k; p.block_tables = st.ws_table; p.max_num_blocks = l.blocks_per_seq;
  p.block_size = kStageBlock; p.num_blocks = (int64_t)num_seqs * l.blocks_per_seq;
  p.block_magic = 0; p.block_bytes = 0; p.num_blocks32 = 0;
  p.timeline = nullptr; p.timeline_entries = 0; p.timeline_block = 0;
  return launch_prefill_pp(p, dtype, s);
}
