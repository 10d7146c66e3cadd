// Varlen causal flash-attention prefill for gfx950.
// Replaces the Triton kernel of src/myvllm/layers/attention.py:111-209.
//
// Packed ragged batch: sequence s owns rows [cu[s], cu[s+1]).  A query tile is
// BM consecutive rows of one sequence; tiles are numbered sequence by sequence
// and a workgroup finds its (sequence, local tile) by walking cu_seqlens, so
// the grid needs only total_tokens and num_seqs (upper bound
// total_tokens/BM + num_seqs tiles) and no host-side maximum length.
#include "common.h"

namespace mvllm {

struct PrefillArgs {
  void* out;
  const void* q;
  const void* k;
  const void* v;
  const int32_t* cu_seqlens;
  int64_t total_tokens;
  int num_seqs;
  int num_heads;
  int num_kv_heads;
  int head_dim;
  float scale_log2;
};

// Tile `tile` (global numbering) -> sequence and first row inside it.
__device__ __forceinline__ bool locate_tile(const int32_t* __restrict__ cu, int num_seqs, int tile, int bm,
                                            int& seq_start, int& seq_len, int& row0) {
  int first = 0;
  int prev = cu[0];
  for (int s = 0; s < num_seqs; ++s) {
    const int next = cu[s + 1];
    const int len = next - prev;
    const int n = (len + bm - 1) / bm;
    if (tile < first + n) {
      seq_start = prev;
      seq_len = len;
      row0 = (tile - first) * bm;
      return true;
    }
    first += n;
    prev = next;
  }
  return false;
}

// ---------------------------------------------------------------------------
// Generic path: any element type, head_dim <= 512.  One wave per query row,
// lanes split head_dim, one key per step.  Correctness path (fp32 inputs and
// head dims the MFMA kernel is not built for).
// ---------------------------------------------------------------------------
constexpr int kGenRows = 16;   // query rows per workgroup (4 waves x 4 rows)
constexpr int kGenMaxR = 8;

template <typename T>
__global__ __launch_bounds__(256) void prefill_generic_kernel(const PrefillArgs a) {
  int seq_start, seq_len, row0;
  if (!locate_tile(a.cu_seqlens, a.num_seqs, blockIdx.x, kGenRows, seq_start, seq_len, row0)) return;
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
    for (int j = 0; j <= r; ++j) {
      const int64_t base = (int64_t)(seq_start + j) * kvrow + (int64_t)g * D;
      float vv[kGenMaxR];
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < kGenMaxR; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
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
    const float linv = 1.f / l;
#pragma unroll
    for (int i = 0; i < kGenMaxR; ++i) {
      const int d = lane + 64 * i;
      if (d < D) op[d] = from_float<T>(acc[i] * linv);
    }
  }
}

template <typename T>
static int launch_prefill_generic(const PrefillArgs& a, hipStream_t stream) {
  const int64_t tiles = a.total_tokens / kGenRows + a.num_seqs;
  prefill_generic_kernel<T><<<dim3((unsigned)tiles, (unsigned)a.num_heads), dim3(256), 0, stream>>>(a);
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

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
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case MVLLM_F32: return launch_prefill_generic<float>(a, s);
    case MVLLM_BF16: return launch_prefill_generic<bf16_t>(a, s);
    default: return launch_prefill_generic<f16_t>(a, s);
  }
}
