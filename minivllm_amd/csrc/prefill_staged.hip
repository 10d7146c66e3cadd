// Prefill over a paged cache in two steps: the keys and values of every sequence of the batch are first written into a
// caller-provided workspace laid out as a 16-bit paged cache with blocks of 16 tokens and a block table of its own, then
// the two-group kernel of prefill_pingpong.hip (shapes it does not take: the one-group kernel's 16-bit paged form) runs
// over that cache.  Two uses:
//  * an INT8 cache: a value is dequantised once (code * scale, rounded to the query's 16-bit type: the value the one-step
//    kernel of prefill_mfma.h feeds the matrix unit) instead of once for every 32-row query tile and head slice that
//    walks its tile, which is most of the one-step kernel's time;
//  * a 16-bit cache whose block size is not a multiple of 16 (8, 1, 24 ...), which the MFMA kernels' tile copies cannot
//    walk and which otherwise runs on the generic kernel.
// No counterpart in the reference (its Triton prefill never reads the paged cache, attention.py:111-209).
#include "common.h"
#include "prefill_mfma.h"

namespace mvllm {

namespace {

constexpr int kStageBlock = 16;        // tokens per block of the staged cache

struct StageArgs {
  const void* k_src;       // codes (int8) or values (16 bit) [num_blocks, block_size, Hkv, D]
  const void* v_src;
  const float* k_scale;    // INT8 source only: [num_blocks, block_size, Hkv]
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

// One workgroup per (16-token block of the staged cache, sequence): its tokens' keys and values, each looked up through
// the source block table, and the block's entry of the staged block table.  A source block whose table entry is not a
// block of the pool reads as zeros, as in the one-step kernels.  Tokens past the sequence's last key are not written
// (the prefill kernels' copy descriptors end with the last key).  A thread moves 16 elements of K and of V at a time.
template <typename T, bool INT8>
__global__ __launch_bounds__(256) void stage_blocks_kernel(const StageArgs a) {
  const int s = blockIdx.y, blk = blockIdx.x;
  const int staged = s * a.blocks_per_seq + blk;
  if (threadIdx.x == 0) a.ws_table[staged] = staged;
  const int kv_len = a.cu_seqlens_k[s + 1] - a.cu_seqlens_k[s];
  const int t0 = kStageBlock * blk;
  if (t0 >= kv_len) return;
  const int row_elems = a.num_kv_heads * a.head_dim;
  const int chunks = row_elems / 16;                           // 16 elements: 16 bytes of codes or 32 bytes of values
  const int rows = kv_len - t0 < kStageBlock ? kv_len - t0 : kStageBlock;
  char* dk = reinterpret_cast<char*>(a.ws_k) + (int64_t)staged * kStageBlock * row_elems * 2;
  char* dv = reinterpret_cast<char*>(a.ws_v) + (int64_t)staged * kStageBlock * row_elems * 2;
  const int32_t* table = a.block_tables + (int64_t)s * a.max_num_blocks;
  for (int idx = threadIdx.x; idx < rows * chunks; idx += 256) {
    const int r = idx / chunks, c = idx - r * chunks;
    const int t = t0 + r;
    const int bi = t / a.block_size, off = t - bi * a.block_size;
    const int phys = bi < a.max_num_blocks ? table[bi] : -1;
    uint4 k0 = make_uint4(0u, 0u, 0u, 0u), k1 = k0, v0 = k0, v1 = k0;
    if (phys >= 0 && (int64_t)phys < a.num_blocks) {
      const int64_t row = (int64_t)phys * a.block_size + off;
      if constexpr (INT8) {
        const int kvh = 16 * c / a.head_dim;
        const float ks = a.k_scale[row * a.num_kv_heads + kvh], vs = a.v_scale[row * a.num_kv_heads + kvh];
        const uint4 ck = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.k_src) + row * row_elems + 16 * c);
        const uint4 cv = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.v_src) + row * row_elems + 16 * c);
        k0 = dequant8_biased<T>(ck.x, ck.y, ks, -128.f * ks);
        k1 = dequant8_biased<T>(ck.z, ck.w, ks, -128.f * ks);
        v0 = dequant8_biased<T>(cv.x, cv.y, vs, -128.f * vs);
        v1 = dequant8_biased<T>(cv.z, cv.w, vs, -128.f * vs);
      } else {
        const uint4* ksrc = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.k_src) + (row * row_elems + 16 * c) * 2);
        const uint4* vsrc = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.v_src) + (row * row_elems + 16 * c) * 2);
        k0 = ksrc[0]; k1 = ksrc[1];
        v0 = vsrc[0]; v1 = vsrc[1];
      }
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

// Which kernel runs over the staged cache: 3 the two-group kernel, 2 the one-group kernel at head_dim 64 / 128, 1 the
// one-group kernel at another head_dim (16-bit sources only), 0: this form is not built for the shape.
int staged_kind(int num_seqs, int max_kv_len, int num_heads, int num_kv_heads, int head_dim, int dtype, bool int8) {
  if (num_seqs <= 0 || max_kv_len <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  if (num_heads > 65535 || dtype == MVLLM_F32 || dtype_size(dtype) == 0) return 0;
  if ((int64_t)num_seqs * ((max_kv_len + kStageBlock - 1) / kStageBlock) >= ((int64_t)1 << 31)) return 0;
  if ((int64_t)num_kv_heads * head_dim * 64 >= ((int64_t)1 << 31)) return 0;
  if (head_dim == 128 || head_dim == 64)
    return prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, kStageBlock) ? 3 : 2;
  return !int8 && prefill_mfma_other_dim(head_dim) ? 1 : 0;
}

int run_staged(void* out, const void* q, const void* k_src, const void* v_src, const float* k_scale, const float* v_scale,
               bool int8, const int32_t* block_tables, int max_num_blocks, const int32_t* cu_seqlens_q,
               const int32_t* cu_seqlens_k, int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
               int num_kv_heads, int head_dim, int block_size, int64_t num_blocks, float scale, int dtype, void* workspace,
               size_t workspace_bytes, void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_q_tokens < 0 || max_kv_len < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 ||
      block_size <= 0 || num_blocks < 0 || max_num_blocks < 0 || num_heads % num_kv_heads != 0 || !(scale > 0.f))
    return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_q_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k_src || !v_src || (int8 && (!k_scale || !v_scale)) || !block_tables || !cu_seqlens_q || !cu_seqlens_k)
    return MVLLM_ERR_NULL_POINTER;
  const int kind = staged_kind(num_seqs, max_kv_len, num_heads, num_kv_heads, head_dim, dtype, int8);
  if (total_q_tokens > ((int64_t)1 << 30) || kind == 0) return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(out) || !aligned16(k_src) || !aligned16(v_src)) return MVLLM_ERR_MISALIGNED;
  const StageLayout l = stage_layout(num_seqs, max_kv_len, num_kv_heads, head_dim);
  if (!workspace || workspace_bytes < l.total_bytes || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return MVLLM_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  StageArgs st;
  st.k_src = k_src; st.v_src = v_src; st.k_scale = k_scale; st.v_scale = v_scale;
  st.block_tables = block_tables; st.cu_seqlens_k = cu_seqlens_k;
  st.ws_k = workspace;
  st.ws_v = reinterpret_cast<char*>(workspace) + l.cache_bytes;
  st.ws_table = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + 2 * l.cache_bytes);
  st.num_blocks = num_blocks; st.max_num_blocks = max_num_blocks; st.block_size = block_size;
  st.num_kv_heads = num_kv_heads; st.head_dim = head_dim; st.blocks_per_seq = l.blocks_per_seq;
  const dim3 grid((unsigned)l.blocks_per_seq, (unsigned)num_seqs), block(256);
  if (dtype == MVLLM_BF16) {
    if (int8) stage_blocks_kernel<bf16_t, true><<<grid, block, 0, s>>>(st);
    else stage_blocks_kernel<bf16_t, false><<<grid, block, 0, s>>>(st);
  } else {
    if (int8) stage_blocks_kernel<f16_t, true><<<grid, block, 0, s>>>(st);
    else stage_blocks_kernel<f16_t, false><<<grid, block, 0, s>>>(st);
  }
  const int status = launch_status();
  if (status != MVLLM_OK) return status;
  const int64_t staged_blocks = (int64_t)num_seqs * l.blocks_per_seq;
  if (kind != 3) {
    PrefillArgs a;
    a.out = out; a.q = q; a.k = st.ws_k; a.v = st.ws_v; a.cu_seqlens = cu_seqlens_q;
    a.total_tokens = total_q_tokens; a.num_seqs = num_seqs; a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
    a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
    a.cu_seqlens_k = cu_seqlens_k; a.block_tables = st.ws_table; a.max_num_blocks = l.blocks_per_seq;
    a.block_size = kStageBlock; a.num_blocks = staged_blocks; a.k_scale = nullptr; a.v_scale = nullptr;
    return kind == 2 ? launch_prefill_paged_16bit(a, dtype, s) : launch_prefill_mfma_other(a, dtype, true, s);
  }
  PrefillPpArgs p;
  p.out = out; p.q = q; p.k = st.ws_k; p.v = st.ws_v; p.cu_seqlens = cu_seqlens_q; p.total_tokens = total_q_tokens;
  p.num_seqs = num_seqs; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.scale_log2 = scale * kLog2e;
  p.slices = 0; p.n_teams = 0; p.team_size = 0; p.level_bits = 0; p.spt_magic = 0; p.chunks_magic = 0;
  p.cu_seqlens_k = cu_seqlens_k; p.block_tables = st.ws_table; p.max_num_blocks = l.blocks_per_seq;
  p.block_size = kStageBlock; p.num_blocks = staged_blocks;
  p.block_magic = 0; p.block_bytes = 0; p.num_blocks32 = 0;
  p.timeline = nullptr; p.timeline_entries = 0; p.timeline_block = 0;
  return launch_prefill_pp(p, dtype, s);
}

}  // namespace

}  // namespace mvllm

using namespace mvllm;

extern "C" size_t mvllm_prefill_paged_staged_workspace_bytes(int num_seqs, int max_kv_len, int num_heads, int num_kv_heads,
                                                             int head_dim, int dtype, int int8_cache) {
  if (staged_kind(num_seqs, max_kv_len, num_heads, num_kv_heads, head_dim, dtype, int8_cache != 0) == 0) return 0;
  return stage_layout(num_seqs, max_kv_len, num_kv_heads, head_dim).total_bytes;
}

extern "C" int mvllm_prefill_paged_staged(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          const int32_t* block_tables, int max_num_blocks, const int32_t* cu_seqlens_q,
                                          const int32_t* cu_seqlens_k, int num_seqs, int64_t total_q_tokens, int max_kv_len,
                                          int num_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                                          float scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  return run_staged(out, q, k_cache, v_cache, nullptr, nullptr, false, block_tables, max_num_blocks, cu_seqlens_q, cu_seqlens_k,
                    num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, dtype,
                    workspace, workspace_bytes, stream);
}

extern "C" int mvllm_prefill_paged_int8_staged(void* out, const void* q, const int8_t* k_cache, const int8_t* v_cache,
                                               const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                               int max_num_blocks, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                               int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                               int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                                               float scale, int dtype, void* workspace, size_t workspace_bytes,
                                               void* stream) {
  return run_staged(out, q, k_cache, v_cache, k_scale, v_scale, true, block_tables, max_num_blocks, cu_seqlens_q, cu_seqlens_k,
                    num_seqs, total_q_tokens, max_kv_len, num_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, dtype,
                    workspace, workspace_bytes, stream);
}
