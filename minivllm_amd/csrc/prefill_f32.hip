// Varlen causal prefill for fp32 tensors (the element type of the reference's demo, main.py:15-41), LDS-tiled:
// replaces the Triton kernel of src/myvllm/layers/attention.py:111-209 for float32 q / k / v with head_dim 128 or 64,
// packed or over a paged fp32 cache.
//
// Same decomposition as prefill_mfma_kernel (prefill_mfma.h): a workgroup of 4 waves is one kv head x 4, 2 or 1 of its
// query heads x 32-row query tiles, K/V tiles shared through LDS by buffer_load ... lds, double-buffered, one barrier
// per tile, items dealt heaviest first.  The arithmetic is v_mfma_f32_32x32x2_f32 (64 clocks per instruction and SIMD,
// 157 TFLOP/s on the data sheet), whose operands are one float per lane:
//   S^T[key][row]  = K Q^T   A = K[key l%32][dim 2s + l/32]  (LDS, rows swizzled by 16-byte chunk),
//                            B = Q[row l%32][dim 2s + l/32]  (registers, scaled by scale * log2 e once)
//   O^T[dim][row] += V^T P^T A = V[key(s, l/32)][dim 32 t + l%32] (LDS, consecutive lanes = consecutive floats),
//                            B = P[row l%32][key(s, l/32)] = the lane's own accumulator register s of S^T
// with key(s, hi) = 8 (s / 4) + 4 hi + s % 4: the order in which a lane's 16 accumulator registers hold the keys of a
// 32 x 32 block, so the weights never leave their registers.  A tile is 32 keys; 128 MFMAs per tile and wave at
// head_dim 128 keep the matrix unit busy for 8192 clocks, against which the softmax's vector work, the LDS reads (one
// dword per MFMA) and the copies are small, so the loop is written plainly: copy the next tile, compute this one.
#include "common.h"
#include "prefill_mfma.h"

namespace mvllm {

namespace {

constexpr int kF32Keys = 32;            // keys per tile

typedef float v16f32 __attribute__((ext_vector_type(16)));

template <int D, int HPW, bool PAGED>
__global__ __launch_bounds__(64 * kPfWaves, 2) void prefill_f32_kernel(const PrefillArgs a) {
  static_assert(D == 128 || D == 64, "head_dim 128 or 64");
  constexpr int kRowB = D * 4;                  // bytes per tile row
  constexpr int kChunks = kRowB / 16;           // 16-byte chunks per row: 32 or 16
  constexpr int kCopyRows = 1024 / kRowB;       // rows per copy instruction: 2 or 4
  constexpr int kTileBytes = kF32Keys * kRowB;  // one K (or V) tile: 16 or 8 KB
  constexpr int ROW_TILES = kPfWaves / HPW;     // 32-row query tiles per workgroup
  constexpr int ROWS_PER_WAVE = kF32Keys / kPfWaves;   // tile rows one wave copies: 8
  constexpr int kCopies = ROWS_PER_WAVE / kCopyRows;   // copy instructions per wave and tile, for K and for V: 4 or 2
  constexpr int BM = kWaveRows * ROW_TILES;     // query rows per workgroup
  constexpr int kSteps = D / 2;                 // 2-dim steps of the first product
  constexpr int kTD = D / 32;                   // 32-dim blocks of the output
  // The 32 lanes of a half-wave read the same chunk of 32 different rows in the first product: the chunk index is
  // xor-ed with the row so that they land in different banks.
  auto swz = [](int row) __attribute__((always_inline)) { return row & (kChunks - 1); };
  struct Tiles { char k[2][kTileBytes]; char v[2][kTileBytes]; };
  __shared__ __attribute__((aligned(1024))) Tiles lds;

  // ---- work item, as in prefill_mfma_kernel ----
  const int tiles_x = a.tiles_x;
  const unsigned id = blockIdx.x;
  const unsigned slot = id >> 3, xcd = id & 7;
  const unsigned round = slot / kXcdChunk;
  const unsigned item = (round * 8 + ((xcd + round) & 7)) * kXcdChunk + slot % kXcdChunk;
  int item_y, seq_start, seq_len, row0, seq_index;
  if (a.num_seqs <= 64) {
    if (!locate_banded<BM>(a.cu_seqlens, a.num_seqs, item, a.heads_y, a.band_bits, a.band_shift, seq_start, seq_len, row0, seq_index, item_y)) return;
  } else {
    if (item >= (unsigned)tiles_x * (unsigned)a.heads_y) return;
    item_y = (int)(item / (unsigned)tiles_x);
    const int item_x = (int)(item % (unsigned)tiles_x);
    if (!locate_tile(a.cu_seqlens, a.num_seqs, tiles_x - 1 - item_x, BM, seq_start, seq_len, row0, seq_index)) return;
  }
  item_y = __builtin_amdgcn_readfirstlane(item_y);
  seq_start = __builtin_amdgcn_readfirstlane(seq_start);
  seq_len = __builtin_amdgcn_readfirstlane(seq_len);
  row0 = __builtin_amdgcn_readfirstlane(row0);
  seq_index = __builtin_amdgcn_readfirstlane(seq_index);
  const int kv_len = PAGED ? a.cu_seqlens_k[seq_index + 1] - a.cu_seqlens_k[seq_index] : seq_len;
  const int cached = PAGED ? max(kv_len - seq_len, 0) : 0;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int group = a.num_heads / a.num_kv_heads;
  const int chunks = group / HPW;
  const int g = item_y / chunks;                                      // kv head
  const int h = g * group + (item_y % chunks) * HPW + (wave % HPW);   // query head of this wave
  const int r0 = row0 + kWaveRows * (wave / HPW);                     // first query row of this wave
  const bool active = r0 < seq_len;
  const int pos0 = cached + r0;                                       // position of that row among the keys
  const int j_last = min(pos0 + kWaveRows - 1, kv_len - 1) / kF32Keys;   // last tile any row of the wave sees
  const int wg_last = min(row0 + BM, seq_len) - 1;
  const int ntiles = (cached + wg_last) / kF32Keys + 1;               // tiles the workgroup walks
  const int l32 = lane & 31;
  const int hi = lane >> 5;
  const int qrow = r0 + l32;                                          // query row of this lane

  const char* kg = reinterpret_cast<const char*>(a.k);
  const char* vg = reinterpret_cast<const char*>(a.v);
  const int row_bytes = a.num_kv_heads * kRowB;
  const int total_rows = (int)a.total_tokens;
  const int rows_4g = (int)(0xffffffffu / (uint32_t)row_bytes);

  // ---- copies: wave w moves rows 8 w .. 8 w + 7 of the K tile and of the V tile ----
  const int ld_row = lane / kChunks, ld_chunk = lane % kChunks;
  uint32_t src_off[kCopies];
#pragma unroll
  for (int i = 0; i < kCopies; ++i) {
    const int row = ROWS_PER_WAVE * wave + kCopyRows * i + ld_row;
    const int src_row = PAGED ? kCopyRows * i + ld_row : row;          // paged: the descriptor starts at the wave's own rows
    src_off[i] = (uint32_t)(src_row * row_bytes + ((ld_chunk ^ swz(row)) << 4));
  }
  const int bs = PAGED ? a.block_size : 1;
  const int32_t* table = PAGED ? a.block_tables + (int64_t)seq_index * a.max_num_blocks : nullptr;
  const uint32_t lds_wave_base = lds_address(&lds.k[0][0]) + (uint32_t)(ROWS_PER_WAVE * wave * kRowB);
  // Tile j -> buffer `buf`.  Packed: the descriptor starts at the tile's first row and ends with the tensor, so rows
  // past the last token arrive as zeros.  Paged: the wave's 8 rows are one piece of one cache block (block_size % 16
  // == 0); the descriptor ends with the sequence's last key; an unmapped block arrives as zeros.
  auto issue_tile = [&](int j, int buf) {
    v4i rk, rv;
    if constexpr (PAGED) {
      const int pos = kF32Keys * j + ROWS_PER_WAVE * wave;
      const int bi = pos / bs, off = pos - bi * bs;
      const int phys = bi < a.max_num_blocks ? table[bi] : -1;
      const int valid = min(ROWS_PER_WAVE, kv_len - pos);
      const bool ok = valid > 0 && phys >= 0 && (int64_t)phys < a.num_blocks;
      const uint32_t size = ok ? (uint32_t)((valid - 1) * row_bytes + kRowB) : 0u;
      const int64_t start = ok ? ((int64_t)phys * bs + off) * row_bytes + (int64_t)g * kRowB : 0;
      rk = make_rsrc(kg + start, size);
      rv = make_rsrc(vg + start, size);
    } else {
      const int first = seq_start + j * kF32Keys;
      const int rows_left = total_rows - first;
      const uint32_t size = rows_left <= 0        ? 0u
                            : rows_left > rows_4g ? 0xffffffffu
                                                  : (uint32_t)rows_left * (uint32_t)row_bytes - (uint32_t)(g * kRowB);
      const int64_t start = (int64_t)first * row_bytes + (int64_t)g * kRowB;
      rk = make_rsrc(kg + start, size);
      rv = make_rsrc(vg + start, size);
    }
    const uint32_t base = lds_wave_base + (uint32_t)buf * kTileBytes;
    static_for<kCopies>([&](auto I) {
      constexpr int i = decltype(I)::value;
      dma16_to_lds<i * 1024>(rk, src_off[i], base);
      dma16_to_lds<2 * kTileBytes + i * 1024>(rv, src_off[i], base);
    });
  };
  issue_tile(0, 0);

  // ---- Q: this lane's row, dims 2 s + hi, times scale * log2 e ----
  float qf[kSteps];
  {
    const float* q = reinterpret_cast<const float*>(a.q);
    int64_t tok = (int64_t)seq_start + qrow;
    if (tok > a.total_tokens - 1) tok = a.total_tokens - 1;            // rows past the tensor: any finite values
    const float2* src = reinterpret_cast<const float2*>(q + (tok * a.num_heads + h) * D);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const float2 x = src[s];
      qf[s] = (hi ? x.y : x.x) * a.scale_log2;
    }
  }

  v16f32 o[kTD];
#pragma unroll
  for (int t = 0; t < kTD; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
  float m = -INFINITY, l = 0.f;                  // running maximum (log2 units) and this lane's share of the row sum

  // per-lane LDS offsets: K rows are read at (row l32, dim 2 s + hi), V rows at (key(s, hi), dim 32 t + l32)
  const int k_row_off = l32 * kRowB;
  const int k_swz = swz(l32);

  for (int j = 0; j < ntiles; ++j) {
    dma_wait_all();
    __syncthreads();                             // tile j has landed; everybody is done with tile j - 1
    if (j + 1 < ntiles) issue_tile(j + 1, (j + 1) & 1);
    if (!active || j > j_last) continue;
    const char* kt = &lds.k[j & 1][0];
    const char* vt = &lds.v[j & 1][0];
    // ---- S^T = K Q^T ----
    // head_dim 128: two accumulators, even and odd steps, so that an MFMA does not wait for the one issued just before
    // it (+6 %; at head_dim 64 the sixteen additions that join them cost more than the 32 steps gain: -10 %)
    constexpr bool kTwoAcc = D == 128;
    v16f32 s, s_odd;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = s_odd[r] = 0.f;
#pragma unroll
    for (int st = 0; st < kSteps; ++st) {
      const int d = 2 * st;                       // dims d, d + 1: chunk d / 4, float (d % 4) + hi inside it
      const float kv = *reinterpret_cast<const float*>(kt + k_row_off + ((((d >> 2) ^ k_swz) << 4) | (((d & 3) + hi) << 2)));
      if (kTwoAcc && (st & 1)) s_odd = __builtin_amdgcn_mfma_f32_32x32x2f32(kv, qf[st], s_odd, 0, 0, 0);
      else s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv, qf[st], s, 0, 0, 0);
    }
    if constexpr (kTwoAcc) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] += s_odd[r];
    }
    // ---- causal mask: key 32 j + 8 (r / 4) + 4 hi + r % 4 against position cached + qrow ----
    if (kF32Keys * j + kF32Keys - 1 > pos0) {
      const int lim = cached + qrow - kF32Keys * j - 4 * hi;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (8 * (r >> 2) + (r & 3) > lim) s[r] = -INFINITY;
    }
    // ---- online softmax ----
    float mx = s[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = max_with_lane_xor32(mx);
    const float m_new = fmaxf(m, mx);
    const float alpha = fast_exp2(m - m_new);    // m = -inf at the first tile: 0
    m = m_new;
    l *= alpha;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      s[r] = fast_exp2(s[r] - m_new);
      sum += s[r];
    }
    l += sum;
    if (alpha != 1.f) {
#pragma unroll
      for (int t = 0; t < kTD; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
    }
    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int st = 0; st < 16; ++st) {
      const int key = 8 * (st >> 2) + 4 * hi + (st & 3);
      const char* vrow = vt + key * kRowB;
      const int vs = swz(key);
#pragma unroll
      for (int t = 0; t < kTD; ++t) {
        const int d = 32 * t + l32;
        const float vv = *reinterpret_cast<const float*>(vrow + ((((d >> 2) ^ vs) << 4) | ((d & 3) << 2)));
        o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, s[st], o[t], 0, 0, 0);
      }
    }
  }

  // ---- output: lane (row l32, hi) holds dims 32 t + 8 (r / 4) + 4 hi + r % 4 ----
  const float row_sum = sum_with_lane_xor32(l);   // (every lane takes part in the exchange)
  if (active && qrow < seq_len) {
    const float inv = 1.f / row_sum;
    float* dst = reinterpret_cast<float*>(a.out) + ((int64_t)(seq_start + qrow) * a.num_heads + h) * D;
#pragma unroll
    for (int t = 0; t < kTD; ++t)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *reinterpret_cast<float4*>(dst + 32 * t + 8 * r4 + 4 * hi) =
            make_float4(o[t][4 * r4] * inv, o[t][4 * r4 + 1] * inv, o[t][4 * r4 + 2] * inv, o[t][4 * r4 + 3] * inv);
  }
}

template <int D, bool PAGED>
int launch_f32_as(const PrefillArgs& a, hipStream_t stream) {
  const int group = a.num_heads / a.num_kv_heads;
  const int hpw = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
  const int bm = kWaveRows * (kPfWaves / hpw);
  PrefillArgs b = a;
  b.band_shift = band_shift_for(a.total_tokens, a.num_seqs, bm, PAGED);
  b.tiles_x = a.num_seqs <= 64 ? (int)(a.total_tokens / bm + ((int64_t)a.num_seqs << b.band_shift))
                               : (int)(a.total_tokens / bm + a.num_seqs);
  b.heads_y = a.num_kv_heads * (group / hpw);
  b.band_bits = 1;
  while (((int64_t)1 << b.band_bits) <= a.total_tokens / (bm << b.band_shift) + 1) ++b.band_bits;
  const int64_t items = (int64_t)b.tiles_x * b.heads_y;
  const int64_t span = 8 * (int64_t)kXcdChunk;
  const dim3 grid((unsigned)((items + span - 1) / span * span)), block(64 * kPfWaves);
  if (hpw == 4) prefill_f32_kernel<D, 4, PAGED><<<grid, block, 0, stream>>>(b);
  else if (hpw == 2) prefill_f32_kernel<D, 2, PAGED><<<grid, block, 0, stream>>>(b);
  else prefill_f32_kernel<D, 1, PAGED><<<grid, block, 0, stream>>>(b);
  return launch_status();
}

}  // namespace

// fp32 q / k / v (and fp32 paged cache), head_dim 128 or 64; paged: block_size a multiple of 16
int launch_prefill_f32(const PrefillArgs& a, bool paged, hipStream_t stream) {
  if (a.head_dim == 128) return paged ? launch_f32_as<128, true>(a, stream) : launch_f32_as<128, false>(a, stream);
  if (a.head_dim == 64) return paged ? launch_f32_as<64, true>(a, stream) : launch_f32_as<64, false>(a, stream);
  return MVLLM_ERR_UNSUPPORTED;
}

}  // namespace mvllm
