// Varlen causal flash-attention prefill for gfx950.
// Replaces the Triton kernel of src/myvllm/layers/attention.py:111-209.
//
// Packed ragged batch: sequence s owns rows [cu[s], cu[s+1]).  A query tile is
// BM consecutive rows of one sequence; tiles are numbered sequence by sequence
// and a workgroup finds its (sequence, local tile) by walking cu_seqlens, so
// the grid needs only total_tokens and num_seqs (upper bound
// total_tokens/BM + num_seqs tiles) and no host-side maximum length.
#include "prefill_mfma.h"

namespace mvllm {


// ---------------------------------------------------------------------------
// Generic path: any element type, head_dim <= 512.  One wave per query row,
// lanes split head_dim, one key per step.  Correctness path (fp32 inputs and
// head dims the MFMA kernel is not built for).
// ---------------------------------------------------------------------------
constexpr int kGenRows = 16;   // query rows per workgroup (4 waves x 4 rows)
constexpr int kGenMaxR = 8;

template <typename T, bool PAGED>
__global__ __launch_bounds__(256) void prefill_generic_kernel(const PrefillArgs a) {
  int seq_start, seq_len, row0, seq_index;
  if (!locate_tile(a.cu_seqlens, a.num_seqs, blockIdx.x, kGenRows, seq_start, seq_len, row0, seq_index)) return;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int h = blockIdx.y;
  const int D = a.head_dim;
  const int g = h / (a.num_heads / a.num_kv_heads);
  const T* q = reinterpret_cast<const T*>(a.q);
  const T* k = reinterpret_cast<const T*>(a.k);
  const T* v = reinterpret_cast<const T*>(a.v);
  T* out = reinterpret_cast<T*>(a.out);
  const int64_t qrow = (int64_t)a.num_heads * D;
  const int64_t kvrow = (int64_t)a.num_kv_heads * D;
  // paged: keys 0 .. cached + r of the sequence, looked up through its block table row
  const int cached = PAGED ? (a.cu_seqlens_k[seq_index + 1] - a.cu_seqlens_k[seq_index]) - seq_len : 0;
  const int32_t* table = PAGED ? a.block_tables + (int64_t)seq_index * a.max_num_blocks : nullptr;

  for (int r = row0 + wave; r < min(row0 + kGenRows, seq_len); r += 4) {
    float qv[kGenMaxR], acc[kGenMaxR];
    const T* qp = q + (int64_t)(seq_start + r) * qrow + (int64_t)h * D;
#pragma unroll
    for (int i = 0; i < kGenMaxR; ++i) {
      const int d = lane + 64 * i;
      qv[i] = d < D ? to_float(qp[d]) : 0.f;
      acc[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    for (int j = 0; j <= cached + r; ++j) {
      int64_t base;
      bool mapped = true;
      if (PAGED) {
        const int bi = j / a.block_size;
        const int phys = bi < a.max_num_blocks ? table[bi] : -1;
        mapped = phys >= 0 && phys < a.num_blocks;               // an unmapped block reads as zero keys and values
        base = ((int64_t)(mapped ? phys : 0) * a.block_size + (j - bi * a.block_size)) * kvrow + (int64_t)g * D;
      } else {
        base = (int64_t)(seq_start + j) * kvrow + (int64_t)g * D;
      }
      float vv[kGenMaxR];
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < kGenMaxR; ++i) {
        const int d = lane + 64 * i;
        if (d < D && mapped) {
          dot = fmaf(qv[i], to_float(k[base + d]), dot);
          vv[i] = to_float(v[base + d]);
        } else {
          vv[i] = 0.f;
        }
      }
      const float s2 = wave_sum(dot) * a.scale_log2;
      const float m_new = fmaxf(m, s2);
      const float alpha = (m == -INFINITY) ? 0.f : fast_exp2(m - m_new);
      const float p = fast_exp2(s2 - m_new);
      l = l * alpha + p;
#pragma unroll
      for (int i = 0; i < kGenMaxR; ++i) acc[i] = fmaf(p, vv[i], acc[i] * alpha);
      m = m_new;
    }
    T* op = out + (int64_t)(seq_start + r) * qrow + (int64_t)h * D;
    const float linv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int i = 0; i < kGenMaxR; ++i) {
      const int d = lane + 64 * i;
      if (d < D) op[d] = from_float<T>(acc[i] * linv);
    }
  }
}

// ---------------------------------------------------------------------------
// MFMA path: 16-bit inputs, head_dim 128 or 64 (described for 128).
//
// Workgroup = 4 waves = (one kv head, HPW of the query heads that share it,
// 4/HPW consecutive 32-row query tiles); every wave owns 32 query rows of one
// head.  Two workgroups share a CU (64 KB of LDS each), so every SIMD holds two
// waves of different workgroups and one's softmax, prologue or epilogue fills
// the gaps of the other.  All waves of a workgroup walk the same 64-row K/V
// tiles, which are copied from global into LDS once per workgroup
// (buffer_load ... lds, 16 B per lane, double buffered, bounds-checked by the
// buffer descriptor), so K/V traffic is shared by the GQA group inside the tile.
//
// Per wave and K/V tile (all MFMA 32x32x16):
//   S^T[kv][q]  = K (A operand, ds_read_b128 from LDS) x Q^T (B operand, registers)
//                 -> lane l holds query row l%32, kv rows 8*(r/4) + 4*(l/32) + r%4
//   softmax       one query row per lane: no cross-lane work except one
//                 xor-32 max; base-2, lazy rescale
//   O^T[d][q]  += V^T (A operand, ds_read_b64_tr_b16 transposing loads) x P^T
//                 (B operand = the S^T accumulators packed to 16 bit in place)
// The contraction index of the second product is permuted so that P needs no
// data movement: k-slot (l/32, e) of step s is kv = 16 s + 8 (e/4) + 4 (l/32) + e%4.
// LDS rows are 256 B; 16-byte chunks are xor-swizzled (K: by row%16, V: by
// 4*(row%4)) so both access patterns spread over all banks.  Causal tiles past
// the diagonal are never visited; only the diagonal tile is masked.
// ---------------------------------------------------------------------------
template <typename T, bool PAGED>
static int launch_prefill_generic(const PrefillArgs& a, hipStream_t stream) {
  const int64_t tiles = a.total_tokens / kGenRows + a.num_seqs;
  prefill_generic_kernel<T, PAGED><<<dim3((unsigned)tiles, (unsigned)a.num_heads), dim3(256), 0, stream>>>(a);
  return launch_status();
}

template <bool PAGED>
static int prefill_dispatch(const PrefillArgs& a, int dtype, bool mfma_ok, hipStream_t s) {
  if (mfma_ok) {
    if (prefill_mfma_other_dim(a.head_dim)) return launch_prefill_mfma_other(a, dtype, PAGED, s);
    return dtype == MVLLM_BF16 ? launch_prefill_mfma<bf16_t, PAGED>(a, s) : launch_prefill_mfma<f16_t, PAGED>(a, s);
  }
  switch (dtype) {
    case MVLLM_F32: return launch_prefill_generic<float, PAGED>(a, s);
    case MVLLM_BF16: return launch_prefill_generic<bf16_t, PAGED>(a, s);
    default: return launch_prefill_generic<f16_t, PAGED>(a, s);
  }
}

}  // namespace mvllm

namespace mvllm {
int launch_prefill_paged_16bit(const PrefillArgs& a, int dtype, hipStream_t stream) {
  return dtype == MVLLM_BF16 ? launch_prefill_mfma<bf16_t, true, false>(a, stream) : launch_prefill_mfma<f16_t, true, false>(a, stream);
}
int launch_prefill_paged_int8(const PrefillArgs& a, int dtype, hipStream_t stream) {
  return dtype == MVLLM_BF16 ? launch_prefill_mfma<bf16_t, true, true>(a, stream) : launch_prefill_mfma<f16_t, true, true>(a, stream);
}
}  // namespace mvllm

using namespace mvllm;

// Which kernel serves a prefill of these static sizes, pointers assumed 16-byte aligned: 2 = the LDS-tiled MFMA
// kernel, 1 = the 16-row tile MFMA kernel, 0 = the generic kernel (one key per step: a correctness path), -1 = none.
static int prefill_kernel_for(int num_heads, int num_kv_heads, int head_dim, int block_size, int dtype, bool paged,
                              bool int8_cache) {
  const bool blocks_ok = !paged || block_size % 16 == 0;
  if (int8_cache) {
    if (dtype == MVLLM_F32 || (head_dim != 128 && head_dim != 64) || !blocks_ok) return -1;
    return (int64_t)block_size * num_kv_heads * head_dim < ((int64_t)1 << 31) ? 2 : 1;
  }
  if (dtype != MVLLM_F32 && (head_dim == 128 || head_dim == 64 || prefill_mfma_other_dim(head_dim)) && blocks_ok &&
      (!paged || (int64_t)block_size * num_kv_heads * head_dim * 2 < ((int64_t)1 << 31)))
    return 2;
  // fp32, head_dim 128 or 64: prefill_f32_kernel (a token row's bytes times 32 tile rows fit 32-bit copy offsets)
  if (dtype == MVLLM_F32 && (head_dim == 128 || head_dim == 64) && blocks_ok &&
      (int64_t)num_kv_heads * head_dim * 4 * 64 < ((int64_t)1 << 31) &&
      (!paged || (int64_t)block_size * num_kv_heads * head_dim * 4 < ((int64_t)1 << 31)))
    return 2;
  if (prefill_rows16_takes(head_dim, dtype, false) && blocks_ok && (int64_t)num_kv_heads * head_dim * 64 < ((int64_t)1 << 31))
    return 1;
  return head_dim <= 64 * kGenMaxR ? 0 : -1;
}

extern "C" int mvllm_prefill_plan(int num_heads, int num_kv_heads, int head_dim, int block_size, int dtype,
                                  int int8_cache, int* kernel) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size < 0 || num_heads % num_kv_heads != 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (kernel) *kernel = prefill_kernel_for(num_heads, num_kv_heads, head_dim, block_size, dtype, block_size > 0, int8_cache != 0);
  return MVLLM_OK;
}

extern "C" int mvllm_prefill_varlen(void* out, const void* q, const void* k, const void* v,
                                    const int32_t* cu_seqlens, int num_seqs, int64_t total_tokens,
                                    int num_heads, int num_kv_heads, int head_dim, float scale, int dtype,
                                    void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_tokens < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k || !v || !cu_seqlens) return MVLLM_ERR_NULL_POINTER;
  if (head_dim > 64 * kGenMaxR || num_heads > 65535) return MVLLM_ERR_UNSUPPORTED;
  if (total_tokens > ((int64_t)1 << 30)) return MVLLM_ERR_UNSUPPORTED;
  PrefillArgs a;
  a.out = out; a.q = q; a.k = k; a.v = v; a.cu_seqlens = cu_seqlens;
  a.total_tokens = total_tokens; a.num_seqs = num_seqs; a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
  a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
  a.cu_seqlens_k = nullptr; a.block_tables = nullptr; a.max_num_blocks = 0; a.block_size = 0; a.num_blocks = 0;
  a.k_scale = nullptr; a.v_scale = nullptr;
  const bool aligned = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(out);
  const int kind = aligned ? prefill_kernel_for(num_heads, num_kv_heads, head_dim, 0, dtype, false, false) : 0;
  const bool mfma_ok = kind == 2;
  if (mfma_ok && dtype == MVLLM_F32) return launch_prefill_f32(a, false, (hipStream_t)stream);
  if (mfma_ok && scale > 0.f && prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, 0)) {
    PrefillPpArgs p;
    p.out = out; p.q = q; p.k = k; p.v = v; p.cu_seqlens = cu_seqlens; p.total_tokens = total_tokens;
    p.num_seqs = num_seqs; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.scale_log2 = scale * kLog2e;
    p.slices = 0; p.n_teams = 0; p.team_size = 0; p.level_bits = 0; p.spt_magic = 0; p.chunks_magic = 0;
    p.cu_seqlens_k = nullptr; p.block_tables = nullptr; p.max_num_blocks = 0; p.block_size = 0; p.num_blocks = 0; p.block_magic = 0; p.block_bytes = 0; p.num_blocks32 = 0;
    p.timeline = nullptr; p.timeline_entries = 0; p.timeline_block = 0;
    return launch_prefill_pp(p, dtype, (hipStream_t)stream);
  }
  // fp32, and 16-bit head dims 32, 80, 96, 112 and 256: 16-row tiles on the decode kernel's tile arithmetic (paged_decode.hip)
  if (kind == 1) {
    PrefillRowsArgs r;
    r.out = out; r.q = q; r.k = k; r.v = v; r.cu_seqlens = cu_seqlens; r.total_tokens = total_tokens;
    r.num_seqs = num_seqs; r.num_heads = num_heads; r.num_kv_heads = num_kv_heads; r.scale_log2 = scale * kLog2e;
    r.cu_seqlens_k = nullptr; r.block_tables = nullptr; r.max_num_blocks = 0; r.block_size = 0; r.num_blocks = 0;
    r.k_scale = nullptr; r.v_scale = nullptr;
    return launch_prefill_rows16(r, head_dim, dtype, (hipStream_t)stream);
  }
  return prefill_dispatch<false>(a, dtype, mfma_ok, (hipStream_t)stream);
}

extern "C" int mvllm_prefill_paged(void* out, const void* q, const void* k_cache, const void* v_cache,
                                   const int32_t* block_tables, int max_num_blocks, const int32_t* cu_seqlens_q,
                                   const int32_t* cu_seqlens_k, int num_seqs, int64_t total_q_tokens,
                                   int num_heads, int num_kv_heads, int head_dim, int block_size,
                                   int64_t num_blocks, float scale, int dtype, void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_q_tokens < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 ||
      block_size <= 0 || num_blocks < 0 || max_num_blocks < 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_q_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k_cache || !v_cache || !block_tables || !cu_seqlens_q || !cu_seqlens_k)
    return MVLLM_ERR_NULL_POINTER;
  if (head_dim > 64 * kGenMaxR || num_heads > 65535) return MVLLM_ERR_UNSUPPORTED;
  if (total_q_tokens > ((int64_t)1 << 30)) return MVLLM_ERR_UNSUPPORTED;
  PrefillArgs a;
  a.out = out; a.q = q; a.k = k_cache; a.v = v_cache; a.cu_seqlens = cu_seqlens_q;
  a.total_tokens = total_q_tokens; a.num_seqs = num_seqs; a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
  a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
  a.cu_seqlens_k = cu_seqlens_k; a.block_tables = block_tables; a.max_num_blocks = max_num_blocks;
  a.block_size = block_size; a.num_blocks = num_blocks; a.k_scale = nullptr; a.v_scale = nullptr;
  const bool aligned = aligned16(q) && aligned16(k_cache) && aligned16(v_cache) && aligned16(out);
  const int kind = aligned ? prefill_kernel_for(num_heads, num_kv_heads, head_dim, block_size, dtype, true, false) : 0;
  const bool mfma_ok = kind == 2;
  if (mfma_ok && dtype == MVLLM_F32) return launch_prefill_f32(a, true, (hipStream_t)stream);
  if (mfma_ok && scale > 0.f && prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, block_size)) {
    PrefillPpArgs p;
    p.out = out; p.q = q; p.k = k_cache; p.v = v_cache; p.cu_seqlens = cu_seqlens_q; p.total_tokens = total_q_tokens;
    p.num_seqs = num_seqs; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.scale_log2 = scale * kLog2e;
    p.cu_seqlens_k = cu_seqlens_k; p.block_tables = block_tables; p.max_num_blocks = max_num_blocks;
    p.block_size = block_size; p.num_blocks = num_blocks; p.block_magic = 0; p.block_bytes = 0; p.num_blocks32 = 0;
    p.slices = 0; p.n_teams = 0; p.team_size = 0; p.level_bits = 0; p.spt_magic = 0; p.chunks_magic = 0;
    p.timeline = nullptr; p.timeline_entries = 0; p.timeline_block = 0;
    return launch_prefill_pp(p, dtype, (hipStream_t)stream);
  }
  if (kind == 1) {
    PrefillRowsArgs r;
    r.out = out; r.q = q; r.k = k_cache; r.v = v_cache; r.cu_seqlens = cu_seqlens_q; r.total_tokens = total_q_tokens;
    r.num_seqs = num_seqs; r.num_heads = num_heads; r.num_kv_heads = num_kv_heads; r.scale_log2 = scale * kLog2e;
    r.cu_seqlens_k = cu_seqlens_k; r.block_tables = block_tables; r.max_num_blocks = max_num_blocks;
    r.block_size = block_size; r.num_blocks = num_blocks; r.k_scale = nullptr; r.v_scale = nullptr;
    return launch_prefill_rows16(r, head_dim, dtype, (hipStream_t)stream);
  }
  return prefill_dispatch<true>(a, dtype, mfma_ok, (hipStream_t)stream);
}

extern "C" int mvllm_prefill_paged_int8(void* out, const void* q, const int8_t* k_cache, const int8_t* v_cache,
                                        const float* k_scale, const float* v_scale, const int32_t* block_tables,
                                        int max_num_blocks, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                        int num_seqs, int64_t total_q_tokens, int num_heads, int num_kv_heads,
                                        int head_dim, int block_size, int64_t num_blocks, float scale, int dtype,
                                        void* stream) {
  if (dtype_size(dtype) == 0) return MVLLM_ERR_BAD_DTYPE;
  if (num_seqs < 0 || total_q_tokens < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 ||
      block_size <= 0 || num_blocks < 0 || max_num_blocks < 0)
    return MVLLM_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return MVLLM_ERR_BAD_SHAPE;
  if (num_seqs == 0 || total_q_tokens == 0) return MVLLM_OK;
  if (!out || !q || !k_cache || !v_cache || !k_scale || !v_scale || !block_tables || !cu_seqlens_q || !cu_seqlens_k)
    return MVLLM_ERR_NULL_POINTER;
  if (dtype == MVLLM_F32 || (head_dim != 128 && head_dim != 64) || block_size % 16 != 0 || num_heads > 65535 ||
      total_q_tokens > ((int64_t)1 << 30) || (int64_t)num_kv_heads * head_dim * 64 >= ((int64_t)1 << 31))
    return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(q) || !aligned16(out) || !aligned16(k_cache) || !aligned16(v_cache)) return MVLLM_ERR_MISALIGNED;
  if (prefill_kernel_for(num_heads, num_kv_heads, head_dim, block_size, dtype, true, true) == 2) {
    PrefillArgs a;
    a.out = out; a.q = q; a.k = k_cache; a.v = v_cache; a.cu_seqlens = cu_seqlens_q;
    a.total_tokens = total_q_tokens; a.num_seqs = num_seqs; a.num_heads = num_heads;
    a.num_kv_heads = num_kv_heads; a.head_dim = head_dim; a.scale_log2 = scale * kLog2e;
    a.tiles_x = 0; a.heads_y = 0; a.band_bits = 0;
    a.cu_seqlens_k = cu_seqlens_k; a.block_tables = block_tables; a.max_num_blocks = max_num_blocks;
    a.block_size = block_size; a.num_blocks = num_blocks; a.k_scale = k_scale; a.v_scale = v_scale;
    return launch_prefill_paged_int8(a, dtype, (hipStream_t)stream);
  }
  PrefillRowsArgs r;
  r.out = out; r.q = q; r.k = k_cache; r.v = v_cache; r.cu_seqlens = cu_seqlens_q; r.total_tokens = total_q_tokens;
  r.num_seqs = num_seqs; r.num_heads = num_heads; r.num_kv_heads = num_kv_heads; r.scale_log2 = scale * kLog2e;
  r.cu_seqlens_k = cu_seqlens_k; r.block_tables = block_tables; r.max_num_blocks = max_num_blocks;
  r.block_size = block_size; r.num_blocks = num_blocks; r.k_scale = k_scale; r.v_scale = v_scale;
  return launch_prefill_rows16(r, head_dim, dtype, (hipStream_t)stream);
}
