// The LDS-tiled MFMA prefill kernel (one group of four waves per workgroup, two workgroups per CU) and its launcher,
// shared by the translation units that instantiate it: prefill_varlen.hip (head_dim 64 and 128, 16-bit and INT8
// caches) and prefill_other_dims.hip (head_dim 32, 80, 96, 112 in the LDS layout of the next of those two).
#pragma once
#include "prefill_tiles.h"

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
  int tiles_x;      // MFMA path: query-tile upper bound (total_tokens / BM + num_seqs)
  int heads_y;      // MFMA path: head slices (kv heads x query-head chunks)
  int band_bits;    // MFMA path: bits that hold the band count of the longest possible sequence (total_tokens / kBandRows + 1)
  // Paged mode (k, v are caches [num_blocks, block_size, Hkv, D]; q holds only the tokens after each
  // sequence's cached prefix): cu_seqlens counts the query rows, cu_seqlens_k the keys (prefix + new).
  const int32_t* cu_seqlens_k;
  const int32_t* block_tables;
  int max_num_blocks;
  int block_size;
  int64_t num_blocks;
  // INT8 cache (paged mode; k, v are int8 codes [num_blocks, block_size, Hkv, D]): fp32 scales
  // [num_blocks, block_size, Hkv], else null
  const float* k_scale;
  const float* v_scale;
  // Paged mode, optional (prefill_split.hip, where one sequence's keys are cut into ranges that are walked as
  // sequences of their own): q_pos = position of each sequence's first query row among its keys where it is not
  // len_k - len_q (a query block that sees all of a key range has q_pos >= len_k); lse = where to write, per (query
  // row, head), log2 of the softmax denominator counted in powers of two (m + log2 l), with which the partial
  // results of the ranges are merged; q_period > 0 = the query tensor holds that many rows and row t of the
  // cu_seqlens numbering reads row t mod q_period (the ranges of a sequence share its queries).  A sequence
  // without keys is skipped.
  const int32_t* q_pos = nullptr;
  float* lse = nullptr;
  int64_t q_period = 0;
  int band_shift = 0;   // MFMA path: log2 of the row tiles per band of the item order (locate_banded)
};

constexpr unsigned kXcdChunk = 32;      // consecutive work items handed to one XCD
constexpr int kPfWaves = 4;             // waves per workgroup: 4, so that two workgroups share a CU
constexpr int kBN = 64;                 // K/V rows per LDS tile
constexpr int kWaveRows = 32;           // query rows per wave

// Eight int8 codes (two dwords, biased by +128 so that the unsigned byte conversions apply) times one scale, rounded
// once to the element type: fma(u, scale, -128 scale) is the exactly rounded (u - 128) * scale = code * scale.
template <typename T> __device__ __forceinline__ uint4 dequant8_biased(uint32_t w0, uint32_t w1, float scale, float bias) {
  const uint32_t u0 = w0 ^ 0x80808080u, u1 = w1 ^ 0x80808080u;
  uint4 r;
  r.x = pack2<T>(fmaf((float)(u0 & 0xffu), scale, bias), fmaf((float)((u0 >> 8) & 0xffu), scale, bias));
  r.y = pack2<T>(fmaf((float)((u0 >> 16) & 0xffu), scale, bias), fmaf((float)(u0 >> 24), scale, bias));
  r.z = pack2<T>(fmaf((float)(u1 & 0xffu), scale, bias), fmaf((float)((u1 >> 8) & 0xffu), scale, bias));
  r.w = pack2<T>(fmaf((float)((u1 >> 16) & 0xffu), scale, bias), fmaf((float)(u1 >> 24), scale, bias));
  return r;
}

// Work item -> (head slice, sequence, first row) for batches of at most 64 sequences, heaviest items first.
// A query tile's cost grows with its position in the sequence (causal: tile t walks t + 1 key tiles), so the items
// are dealt in bands of kBandRows rows: band b of a sequence is its row tiles [b R, b R + R), R = kBandRows / BM.  The order is
// band level descending (every sequence's last band comes before anybody's band below it), inside a level head
// slice, then sequence, then the band's R tiles from the last (heaviest) down.  The launch then ends with the
// level-0 bands of all sequences, whose items take a few key tiles each, instead of with whatever rows the last
// sequence in memory order has: with 16 prompts of 64-2048 tokens the launch used to end with a single prompt's
// 60-tile items running alone.  Consecutive items still share a sequence's keys (R tiles of one band, and
// neighbouring bands of the same level), which keeps them in one XCD's L2.  Bands past a sequence's last tile are
// padding: those workgroups return at once (at most R - 1 per sequence and head slice), which still costs each of
// them a place on a CU for the two microseconds of this function: a packed batch of short prompts (at most 192 rows on
// average) is dealt in bands of one tile (band_shift 0), which have no padding, and whose loss of L2 sharing between
// a sequence's tiles costs such prompts nothing.
// Every lane of the calling wave must be active; all lanes return the same values.
constexpr int kBandRows = 256;          // rows per band of the heaviest-first item order (a multiple of 128)
constexpr int kShortPromptRows = 192;   // mean rows per sequence up to which bands are single tiles
// log2 of the row tiles per band for a batch of these static sizes (bm: rows per workgroup, a power of two <= kBandRows)
// (packed: the rows are also the keys.  Over a cached prefix few rows may stand behind many keys, which the tiles of a
// band share in one XCD's L2: 128 rows behind 32768 keys cut into ranges ran 100 us in single tiles against 88.)
inline int band_shift_for(int64_t total_tokens, int num_seqs, int bm, bool paged) {
  if (!paged && total_tokens <= (int64_t)num_seqs * kShortPromptRows) return 0;
  int shift = 0;
  while ((bm << shift) < kBandRows) ++shift;
  return shift;
}
template <int BM>
__device__ __forceinline__ bool locate_banded(const int32_t* __restrict__ cu, int num_seqs, unsigned item, int heads_y,
                                              int band_bits, int band_shift, int& seq_start, int& seq_len, int& row0, int& seq_index,
                                              int& item_y) {
  const int R = 1 << band_shift;
  const int lane = threadIdx.x & 63;
  int lo = 0, len = 0;
  if (lane < num_seqs) {
    lo = cu[lane];
    len = cu[lane + 1] - lo;
  }
  const int n = (len + BM - 1) / BM;            // row tiles of the lane's sequence
  const int nb = (n + R - 1) >> band_shift;     // ... and bands
  // highest band level in the batch: bit by bit from the top (band_bits: the host's bound from the token count)
  int top = 0;
  for (int bit = band_bits - 1; bit >= 0; --bit) {
    const int trial = top | (1 << bit);
    if (__ballot(nb >= trial) != 0ull) top = trial;
  }
  // walk the levels down from the top one until the item's level is found
  unsigned base = 0;
  int b = top - 1;
  unsigned long long mask = 0ull;
  unsigned per_y = 0;
  for (; b >= 0; --b) {
    mask = __ballot(nb > b);
    per_y = (unsigned)__popcll(mask) << band_shift;
    const unsigned items = per_y * (unsigned)heads_y;
    if (item - base < items) break;
    base += items;
  }
  if (b < 0) return false;                      // past the last item: grid padding
  const unsigned idx = item - base;
  item_y = (int)(idx / per_y);
  const unsigned rem = idx - (unsigned)item_y * per_y;
  const int q = (int)(rem >> band_shift), r = (int)(rem & (unsigned)(R - 1));
  // the q-th sequence of this level = the lane whose bit is set with q set bits below it
  const int below = __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
  const unsigned long long pick = __ballot(((mask >> lane) & 1ull) != 0ull && below == q);
  const int owner = __ffsll((long long)pick) - 1;
  const int t = (b << band_shift) + (R - 1 - r);   // row tile inside the sequence, last tile of the band first
  if (t >= __shfl(n, owner, 64)) return false;  // the band's padding
  seq_start = __shfl(lo, owner, 64);
  seq_len = __shfl(len, owner, 64);
  row0 = t * BM;
  seq_index = owner;
  return true;
}

// D = 256, 128 or 64.  A row of a tile is D*2 bytes = kChunks 16-byte chunks; one copy instruction moves 1 KB = kCopyRows
// rows.  The chunk swizzles (kswz for K, vswz for V) must not change when 8, 16 or 32 rows are added, because the
// per-lane LDS offsets are computed once and the tile rows are reached through immediates.
// I8 (paged only): the cache holds int8 codes and fp32 scales per (token, kv head).  The codes of a tile are copied
// into a staging area of LDS (the second K and V buffers, two tiles of codes each), and every wave dequantises its
// 16 rows into the one 16-bit K and V tile (code * scale rounded once to the element type, exactly what the 16-row
// tile kernel and decode see), after which the tile is an ordinary tile: two barriers per tile instead of one, the
// conversion (about 180 vector instructions per lane and tile) in front of the products.
// DD (default D): the head dimension of the data where it is not 64, 128 or 256 itself: 32 to 56 in the layout of 64,
// 72 to 120 in that of 128, in steps of 8.  A tile row is still copied as D * 2 bytes, so its last chunks hold whatever
// follows the head in memory (the next head, the next token, zeros past the descriptor's end); the first product runs
// over ceil(DD / 16) steps and never reads them (kHalfStep below: the last step of DD = 16 n + 8), the second one
// carries them through the output columns DD .. 32 ceil(DD / 32) - 1 of its last block, which are not stored.
template <typename T, int HPW, bool PAGED, int D, bool I8 = false, int DD = D>
__global__ __launch_bounds__(64 * kPfWaves, D == 256 ? 1 : 2) void prefill_mfma_kernel(const PrefillArgs a) {
  static_assert(!I8 || PAGED, "INT8 caches are paged");
  static_assert(DD % 8 == 0 && DD <= D && (!I8 || DD == D), "head dims in steps of 8, INT8 only at 64 and 128");
  constexpr int kRowB = D * 2;                  // bytes per tile row
  constexpr int kChunks = kRowB / 16;           // 16-byte chunks per row: 16 or 8
  constexpr int kCopyRows = 1024 / kRowB;       // rows per copy instruction: 4 or 8
  constexpr int kTileBytes = kBN * kRowB;       // one K (or V) tile
  constexpr int kKS = (DD + 15) / 16;           // 16-dim steps of the first product
  // DD = 16 n + 8: the last step holds 8 dims.  Its upper lanes (hi = 1, dims 8 .. 15 of the step) carry zeros as Q and
  // read the row's first chunk as K (data of the same row and head, so the products are exact zeros and nothing of the
  // neighbouring head is touched).
  constexpr bool kHalfStep = DD % 16 == 8;
  constexpr int kTD = (DD + 31) / 32;           // 32-dim blocks of the output
  // K rows are read 16 at a time with the same logical chunk: the swizzle spreads them over the banks.  With 128-byte
  // rows two rows share a 256-byte bank line, so the row index is halved first.
  auto kswz = [](int row) __attribute__((always_inline)) { return D >= 128 ? (row & 15) : ((row >> 1) & 7); };
  // V is read by the transposing loads as 4 rows x 64 bytes per 16 lanes: bits 2-3 of the chunk index take the row's
  // low bits so that the four rows land in four 64-byte groups.  Bit 0 (D = 128) swaps the chunks of a pair in odd
  // rows; the reads do not care (the pair stays in its group), and the INT8 conversion's LDS writes, which go two rows
  // x four quarters at a time over 128 bytes of banks, meet 2-way instead of 4-way (32 -> 16 clocks per write).
  auto vswz = [](int row) __attribute__((always_inline)) { return D >= 128 ? (((row & 3) << 2) | (row & 1)) : (((row >> 1) & 1) << 2); };
  constexpr int ROW_TILES = kPfWaves / HPW;     // 32-row query tiles per workgroup
  constexpr int ROWS_PER_WAVE = kBN / kPfWaves; // K/V tile rows one wave copies (4 per instruction)
  constexpr int BM = kWaveRows * ROW_TILES;     // query rows per workgroup
  struct Tiles { char k[2][kTileBytes]; char v[2][kTileBytes]; };     // double-buffered K and V tiles
  __shared__ __attribute__((aligned(1024))) Tiles lds;

  // Work item = (head slice y, query tile x), x fastest.  Workgroups are dealt to the 8 XCDs round-robin by
  // linear id; items are handed out in chunks of kXcdChunk consecutive items per XCD so that workgroups
  // sharing one sequence's K/V run on the same XCD (same L2) at about the same time.
  const int tiles_x = a.tiles_x;
  const unsigned id = blockIdx.x;
  const unsigned slot = id >> 3, xcd = id & 7;
  // round q of an XCD takes chunk 8q + (xcd + q) % 8: the rotation spreads the heavy (late-tile) chunks of
  // a long sequence over all XCDs instead of always handing them to the same one
  const unsigned round = slot / kXcdChunk;
  const unsigned item = (round * 8 + ((xcd + round) & 7)) * kXcdChunk + slot % kXcdChunk;
  int item_y, seq_start, seq_len, row0, seq_index;
  if (a.num_seqs <= 64) {
    if (!locate_banded<BM>(a.cu_seqlens, a.num_seqs, item, a.heads_y, a.band_bits, a.band_shift, seq_start, seq_len, row0, seq_index, item_y)) return;
  } else {
    // more sequences than one wave holds: memory order, inside a sequence the latest (heaviest) tiles first
    if (item >= (unsigned)tiles_x * (unsigned)a.heads_y) return;
    item_y = (int)(item / (unsigned)tiles_x);
    const int item_x = (int)(item % (unsigned)tiles_x);
    if (!locate_tile(a.cu_seqlens, a.num_seqs, tiles_x - 1 - item_x, BM, seq_start, seq_len, row0, seq_index)) return;
  }
  item_y = __builtin_amdgcn_readfirstlane(item_y);
  // Wave-uniform by construction; say so, so that everything derived from them (tile counts, loop bounds,
  // tile base addresses, branches) lives in scalar registers and runs on the scalar unit.
  seq_start = __builtin_amdgcn_readfirstlane(seq_start);
  seq_len = __builtin_amdgcn_readfirstlane(seq_len);
  row0 = __builtin_amdgcn_readfirstlane(row0);
  seq_index = __builtin_amdgcn_readfirstlane(seq_index);
  // Keys of the sequence: its own rows, or in paged mode the cached prefix plus them (query row r sits at
  // position cached + r and sees keys 0 .. cached + r).
  const int kv_len = PAGED ? a.cu_seqlens_k[seq_index + 1] - a.cu_seqlens_k[seq_index] : seq_len;
  const int cached = !PAGED ? 0 : a.q_pos != nullptr ? a.q_pos[seq_index] : max(kv_len - seq_len, 0);
  if (PAGED && a.q_pos != nullptr && kv_len <= 0) return;   // a key range that is empty (uniform over the workgroup)

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int group = a.num_heads / a.num_kv_heads;
  const int chunks = group / HPW;                    // workgroups per kv head
  const int g = item_y / chunks;                     // kv head
  const int h = g * group + (item_y % chunks) * HPW + (wave % HPW);   // query head of this wave
  const int r0 = row0 + kWaveRows * (wave / HPW);    // first query row of this wave (inside the sequence)
  const bool active = r0 < seq_len;
  const int pos0 = cached + r0;                      // position of that row among the keys
  // tiles every row of the wave sees completely (a row sees keys up to its position, and never past the last key)
  const int n_full = min((pos0 + 1) / kBN, kv_len / kBN);
  const int j_last = min(pos0 + kWaveRows - 1, kv_len - 1) / kBN;   // last tile any row of the wave sees
  const int wg_last = min(row0 + BM, seq_len) - 1;
  const int ntiles = min((cached + wg_last) / kBN, (kv_len - 1) / kBN) + 1;
  const int l32 = lane & 31;
  const int hi = lane >> 5;                          // 0/1: which half of the k-slots / rows
  const int qrow = r0 + l32;                         // query row of this lane

  const T* q = reinterpret_cast<const T*>(a.q);
  const char* kg = reinterpret_cast<const char*>(a.k);
  const char* vg = reinterpret_cast<const char*>(a.v);
  constexpr int kElt = I8 ? 1 : 2;                    // bytes per cache element
  const int64_t kv_row_bytes = (int64_t)a.num_kv_heads * DD * kElt;
  const int64_t last_token = a.total_tokens - 1;

  // ---- K/V tile DMA: wave w moves ROWS_PER_WAVE rows (4 per instruction) of K and of V.
  // Addresses are a wave-uniform 64-bit base (tile start, SALU arithmetic) plus a per-lane 32-bit offset that
  // never changes, so a tile costs no VALU address math.  Only a tile that runs past the last packed token
  // (the tail of the last sequence) recomputes clamped offsets.
  const int ld_row = lane / kChunks;   // row inside the group of rows one instruction copies
  const int ld_chunk = lane % kChunks; // destination chunk inside the row
  constexpr int kCopies = ROWS_PER_WAVE / kCopyRows;
  static_assert(!PAGED || ROWS_PER_WAVE == 16, "paged mode: one wave copies one 16-row piece of a cache block");
  uint32_t k_src_off[kCopies], v_src_off[kCopies];
#pragma unroll
  for (int i = 0; i < kCopies; ++i) {
    const int row = ROWS_PER_WAVE * wave + kCopyRows * i + ld_row;   // row inside the tile (decides the swizzle)
    const int src_row = PAGED ? kCopyRows * i + ld_row : row;        // paged: the descriptor starts at the wave's own rows
    k_src_off[i] = (uint32_t)(src_row * (int)kv_row_bytes + ((ld_chunk ^ kswz(row)) << 4));
    v_src_off[i] = (uint32_t)(src_row * (int)kv_row_bytes + ((ld_chunk ^ vswz(row)) << 4));
  }
  // INT8: a row of codes is D bytes = D / 16 chunks, one copy instruction moves 1024 / D rows, unswizzled (the
  // staging area is read back linearly); the same offset serves K and V
  constexpr int kChunks8 = D / 16, kCopyRows8 = 1024 / D, kCopies8 = ROWS_PER_WAVE / kCopyRows8;
  uint32_t c_src_off[kCopies8];
#pragma unroll
  for (int i = 0; i < kCopies8; ++i)
    c_src_off[i] = (uint32_t)((kCopyRows8 * i + lane / kChunks8) * (int)kv_row_bytes + ((lane % kChunks8) << 4));
  // One tile's copy is 2 * kCopies instructions per wave (K copies first, then V).  Inside tile_step they are
  // issued one at a time, spread between the MFMAs of the tile before, because a wave that issues them back
  // to back sits in the memory pipeline's queue instead of feeding the matrix unit.  The descriptor of a tile
  // starts at the tile's first row and ends with the tensor, so rows past the last packed token arrive as
  // zeros; a descriptor of size 0 (enable = false) turns the copy into a zero fill that touches no memory,
  // which keeps the last tile's code free of branches.
  // Paged mode: the wave's 16 rows of a tile are one piece of one cache block (block_size % 16 == 0); the
  // descriptor starts at that piece and ends with the sequence's last key, so rows of the block that were
  // never written (and unmapped blocks) arrive as zeros.  Tiles are asked for in order, once each, so the
  // piece's block index and offset advance by 64 keys per call; block-table entries come from a 64-entry
  // window held one per lane, as in the decode kernel.
  struct TileSrc { v4i k, v; int64_t slot; int valid; };   // slot, valid: INT8 only (first token slot and live rows of the piece)
  const int row_bytes = (int)kv_row_bytes;
  const int total_rows = (int)a.total_tokens;
  const int rows_4g = (int)(0xffffffffu / (uint32_t)row_bytes);   // rows whose bytes no longer fit 32 bits
  const int bs = PAGED ? a.block_size : 1;
  const int32_t* table = PAGED ? a.block_tables + (int64_t)seq_index * a.max_num_blocks : nullptr;
  int pg_pos = ROWS_PER_WAVE * wave;                 // key position of this wave's piece in the next tile asked for
  int pg_bi = pg_pos / bs, pg_off = pg_pos - pg_bi * bs;
  int win_base = 0;
  int win = -1;
  if (PAGED) win = lane < a.max_num_blocks ? table[lane] : -1;
  auto tile_src = [&](int j, bool enable) {
    TileSrc t;
    if constexpr (PAGED) {
      (void)j;
      if (pg_bi - win_base >= 64) {
        win_base = pg_bi;
        win = win_base + lane < a.max_num_blocks ? table[win_base + lane] : -1;
      }
      const int phys = __builtin_amdgcn_readlane(win, pg_bi - win_base);
      const int valid = min(ROWS_PER_WAVE, kv_len - pg_pos);
      const bool ok = enable && valid > 0 && pg_bi < a.max_num_blocks && phys >= 0 && (int64_t)phys < a.num_blocks;
      const uint32_t size = ok ? (uint32_t)((valid - 1) * row_bytes + DD * kElt) : 0u;
      const int64_t start = ok ? ((int64_t)phys * bs + pg_off) * kv_row_bytes + (int64_t)g * (DD * kElt) : 0;
      t.k = make_rsrc(kg + start, size);
      t.v = make_rsrc(vg + start, size);
      t.slot = ok ? (int64_t)phys * bs + pg_off : 0;
      t.valid = ok ? valid : 0;
      pg_pos += kBN;
      pg_off += kBN;
      while (pg_off >= bs) {
        pg_off -= bs;
        ++pg_bi;
      }
    } else {
      const int row0 = seq_start + j * kBN;                          // first row of the tile
      const int rows_left = total_rows - row0;
      const uint32_t size = (!enable || rows_left <= 0) ? 0u
                            : rows_left > rows_4g       ? 0xffffffffu
                                                        : (uint32_t)rows_left * (uint32_t)row_bytes - (uint32_t)(g * (DD * 2));
      const int64_t start = (int64_t)row0 * kv_row_bytes + (int64_t)g * (DD * 2);
      t.k = make_rsrc(kg + start, size);
      t.v = make_rsrc(vg + start, size);
      t.slot = 0;
      t.valid = 0;
    }
    return t;
  };
  // LDS byte address of this wave's first row in buffer 0 of K; V, buffer 1 and later copies are constants away
  // (the two arrays are laid out back to back by the struct below).
  const uint32_t lds_wave_base = lds_address(&lds.k[0][0]) + (uint32_t)(ROWS_PER_WAVE * wave * kRowB);
  auto issue_copy = [&](const TileSrc& t, auto BUF, auto C) {               // C < kCopies: K copy C, else V copy C - kCopies
    constexpr int c = decltype(C)::value;
    constexpr bool is_k = c < kCopies;
    constexpr int i = is_k ? c : c - kCopies;
    constexpr int imm = (is_k ? 0 : 2 * kTileBytes) + decltype(BUF)::value * kTileBytes + i * 1024;
    dma16_to_lds<imm>(is_k ? t.k : t.v, is_k ? k_src_off[i] : v_src_off[i], lds_wave_base);
  };
  auto issue_tile = [&](int j, int buf) {                        // whole tile at once, buffer chosen at run time
    const TileSrc t = tile_src(j, true);
    const uint32_t base = lds_wave_base + (uint32_t)buf * kTileBytes;
    static_for<kCopies>([&](auto I) {
      constexpr int i = decltype(I)::value;
      dma16_to_lds<i * 1024>(t.k, k_src_off[i], base);
      dma16_to_lds<2 * kTileBytes + i * 1024>(t.v, v_src_off[i], base);
    });
  };
  // ---- INT8: codes -> staging (k[1] / v[1], two tiles of codes each), scales -> registers, then conversion
  const uint32_t lds_stage_base = lds_address(&lds.k[1][0]) + (uint32_t)(ROWS_PER_WAVE * wave * D);
  const int cv_row = lane >> 2, cv_quarter = lane & 3;        // conversion: 4 lanes per row of the wave's 16
  struct Scales { float k, v; };
  auto issue_codes = [&](int j, bool enable) {                // codes of tile j -> staging[j & 1]; returns its scales
    const TileSrc t = tile_src(j, enable);
    const uint32_t base = lds_stage_base + (uint32_t)(j & 1) * (kTileBytes / 2);
    static_for<kCopies8>([&](auto I) {
      constexpr int i = decltype(I)::value;
      dma16_to_lds<i * 1024>(t.k, c_src_off[i], base);
      dma16_to_lds<2 * kTileBytes + i * 1024>(t.v, c_src_off[i], base);
    });
    Scales sc = {0.f, 0.f};
    if (cv_row < t.valid) {
      const int64_t at = (t.slot + cv_row) * a.num_kv_heads + g;
      sc.k = a.k_scale[at];
      sc.v = a.v_scale[at];
    }
    return sc;
  };
  auto convert_tile = [&](int j, const Scales& sc) {          // staging[j & 1] -> the 16-bit tile in k[0] / v[0]
    constexpr int kReads = D / 64;                            // 16-byte reads per lane (D / 4 codes)
    const int row = ROWS_PER_WAVE * wave + cv_row;            // row inside the tile
    const char* ks8 = &lds.k[1][0] + (j & 1) * (kTileBytes / 2) + row * D + cv_quarter * (D / 4);
    const char* vs8 = ks8 + 2 * kTileBytes;
    char* kd = &lds.k[0][0] + row * kRowB;
    char* vd = &lds.v[0][0] + row * kRowB;
    const float kb = -128.f * sc.k, vb = -128.f * sc.v;
#pragma unroll
    for (int r = 0; r < kReads; ++r) {
      const uint4 ck = *reinterpret_cast<const uint4*>(ks8 + 16 * r);
      const uint4 cv = *reinterpret_cast<const uint4*>(vs8 + 16 * r);
      const int c = cv_quarter * (2 * kReads) + 2 * r;        // first of the two 16-byte chunks these 16 codes fill
      *reinterpret_cast<uint4*>(kd + (((c) ^ kswz(row)) << 4)) = dequant8_biased<T>(ck.x, ck.y, sc.k, kb);
      *reinterpret_cast<uint4*>(kd + (((c + 1) ^ kswz(row)) << 4)) = dequant8_biased<T>(ck.z, ck.w, sc.k, kb);
      *reinterpret_cast<uint4*>(vd + (((c) ^ vswz(row)) << 4)) = dequant8_biased<T>(cv.x, cv.y, sc.v, vb);
      *reinterpret_cast<uint4*>(vd + (((c + 1) ^ vswz(row)) << 4)) = dequant8_biased<T>(cv.z, cv.w, sc.v, vb);
    }
  };
  Scales sc_cur = {0.f, 0.f};
  if constexpr (I8) sc_cur = issue_codes(0, true);
  else issue_tile(0, 0);

  // Q fragments (B operand): column = query row l32, k = 16*ks + 8*hi ..
  uint4 qf[kKS];
  {
    int64_t tok = (int64_t)seq_start + qrow;
    if (tok > last_token) tok = last_token;
    if (PAGED && a.q_period > 0) tok = (int64_t)((uint32_t)tok % (uint32_t)a.q_period);   // both below 2^31
    const T* src = q + (tok * a.num_heads + h) * DD + 8 * hi;
#pragma unroll
    for (int ks = 0; ks < DD / 16; ++ks) qf[ks] = *reinterpret_cast<const uint4*>(src + 16 * ks);
    if constexpr (kHalfStep) {
      qf[kKS - 1] = make_uint4(0u, 0u, 0u, 0u);
      if (hi == 0) qf[kKS - 1] = *reinterpret_cast<const uint4*>(src + 16 * (kKS - 1));
    }
    // The softmax scale (times log2 e) goes into Q once, rounded to the element type, so that the scores leave
    // the matrix unit as exp2 arguments: the tile loop has no multiply per score.  This runs while the first K/V
    // tile is still on its way.
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
      qf[ks].x = scale_pair<T>(qf[ks].x, a.scale_log2);
      qf[ks].y = scale_pair<T>(qf[ks].y, a.scale_log2);
      qf[ks].z = scale_pair<T>(qf[ks].z, a.scale_log2);
      qf[ks].w = scale_pair<T>(qf[ks].w, a.scale_log2);
    }
  }
  // Make the compiler retire the Q loads here: otherwise it carries "Q may still be in flight" into
  // the loop and its vmcnt waits there would also wait for the tile prefetch.
#pragma unroll
  for (int ks = 0; ks < kKS; ++ks) asm volatile("" ::"v"(qf[ks].x), "v"(qf[ks].w));

  v16f o[kTD];
#pragma unroll
  for (int td = 0; td < kTD; ++td)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[td][r] = 0.f;
  // Running maximum of the lane's query row, kept negated in all 16 registers of an accumulator tuple: the score
  // products start from it (C operand of their first MFMA), so a tile's scores arrive as  s * scale * log2 e - m,
  // ready for exp2.  It only changes when a tile's maximum exceeds it by more than 2^8 (lazy rescale), which
  // is rare after a row's first tile.
  v16f neg_m;
#pragma unroll
  for (int r = 0; r < 16; ++r) neg_m[r] = 0.f;
  bool first = true;                                 // no tile seen yet: the maximum is still the placeholder 0
  float l = 0.f;

  // Per-lane LDS byte offsets, computed once: the xor swizzle keeps the compiler from folding them into
  // instruction offsets, so they live in registers and every LDS read below is base + immediate.
  //   K: row l32 (+32 rows per tk = +8192 B), 16-byte chunk (2*ks + hi) ^ (l32 & 15)
  //   V: row 4*hi + (lane&15)/4 (+8, +16*st, +32*tk rows), chunk (4*td + 2*half + ...) ^ (4*(row & 3) | (row & 1))
  const int i16 = lane & 15;
  const int half = (lane >> 4) & 1;
  // (The swizzles are xors on the low four bits of the chunk index, so with 32 chunks per row (head_dim 256) the
  // offsets of step ks + 8 and block td + 4 are those of ks and td plus 256 bytes: an immediate, not another register.)
  constexpr int kKOffs = kKS > 8 ? 8 : kKS, kVOffs = kTD > 4 ? 4 : kTD;
  int k_off_[kKOffs];
#pragma unroll
  for (int ks = 0; ks < kKOffs; ++ks) k_off_[ks] = l32 * kRowB + (((2 * ks + hi) ^ kswz(l32)) << 4);
  if constexpr (kHalfStep) k_off_[kKS - 1] = l32 * kRowB + (((hi ? 0 : 2 * (kKS - 1)) ^ kswz(l32)) << 4);
  auto k_off = [&](int ks) __attribute__((always_inline)) { return k_off_[ks & 7] + (ks >> 3) * 256; };
  const int v_row = 4 * hi + (i16 >> 2);
  int v_off_[kVOffs];
#pragma unroll
  for (int td = 0; td < kVOffs; ++td)
    v_off_[td] = v_row * kRowB + (((4 * td + 2 * half + ((i16 & 3) >> 1)) ^ vswz(v_row)) << 4) + ((i16 & 1) << 3);
  auto v_off = [&](int td) __attribute__((always_inline)) { return v_off_[td & 3] + (td >> 2) * 256; };

  // One K/V tile: scores, softmax, P.V.  Compile-time parameters: BUF, the buffer index (so that all LDS
  // addresses are register + constant); DIAG, set for the wave's last tile, the one the causal diagonal runs
  // through (the only one that is masked); NH, the number of 32-row halves of the tile that are computed at
  // all: 1 when the wave's rows are the upper half of the 64-row block, so that the diagonal tile's second
  // half is masked entirely.
  auto tile_step = [&](int j, auto BUF, auto DIAG, auto NHALF, bool prefetch) {
    constexpr int buf = decltype(BUF)::value;
    constexpr bool diag = decltype(DIAG)::value;
    constexpr int NH = decltype(NHALF)::value;
    using NEXT_BUF = std::integral_constant<int, buf ^ 1>;
    TileSrc next;
    if constexpr (!I8) next = tile_src(j + 1, prefetch);      // INT8: the codes of the next tile are already on their way

    // ---- S^T = K Q^T (on the diagonal tile rows past the causal limit are computed and then masked) ----
    // The two 32-row halves of the tile form two independent accumulator chains that are issued
    // alternately, so no MFMA waits for the result of the one before it.
    v16f s[NH];
    const char* kb = &lds.k[buf][0];
    {
      // K fragments are read one step ahead of the MFMAs that use them.  The reads of step ks + 1 stand in front
      // of step ks's copy instruction on purpose: the copy is an asm statement, which no LDS read is moved
      // across, so reads placed after it would be issued right before their use and wait out the LDS latency.
      if constexpr (D == 256) {
        // One wave per SIMD: nothing else covers an LDS round trip, so the fragments are requested two steps (four
        // MFMAs) ahead.
        uint4 kf[3][NH];
#pragma unroll
        for (int pre = 0; pre < 2; ++pre)
#pragma unroll
          for (int tk = 0; tk < NH; ++tk) kf[pre][tk] = *reinterpret_cast<const uint4*>(kb + k_off(pre) + tk * 32 * kRowB);
        static_for<kKS>([&](auto KS) {
          constexpr int ks = decltype(KS)::value;
          if constexpr (ks + 2 < kKS) {
#pragma unroll
            for (int tk = 0; tk < NH; ++tk)
              kf[(ks + 2) % 3][tk] = *reinterpret_cast<const uint4*>(kb + k_off(ks + 2) + tk * 32 * kRowB);
            __builtin_amdgcn_sched_barrier(0);
          }
#pragma unroll
          for (int tk = 0; tk < NH; ++tk) s[tk] = mfma32x32x16<T>(kf[ks % 3][tk], qf[ks], ks == 0 ? neg_m : s[tk]);
          if constexpr (!I8 && ks < 2 * kCopies) issue_copy(next, NEXT_BUF{}, KS);
        });
      } else {
        uint4 kf[2][NH];
#pragma unroll
        for (int tk = 0; tk < NH; ++tk) kf[0][tk] = *reinterpret_cast<const uint4*>(kb + k_off(0) + tk * 32 * kRowB);
        static_for<kKS>([&](auto KS) {
          constexpr int ks = decltype(KS)::value;
          if constexpr (ks + 1 < kKS) {
#pragma unroll
            for (int tk = 0; tk < NH; ++tk)
              kf[(ks + 1) & 1][tk] = *reinterpret_cast<const uint4*>(kb + k_off(ks + 1) + tk * 32 * kRowB);
            __builtin_amdgcn_sched_barrier(0);   // keep the reads in front of this step's MFMAs
          }
#pragma unroll
          for (int tk = 0; tk < NH; ++tk) s[tk] = mfma32x32x16<T>(kf[ks & 1][tk], qf[ks], ks == 0 ? neg_m : s[tk]);
          if constexpr (!I8 && ks < 2 * kCopies) issue_copy(next, NEXT_BUF{}, KS);    // copies of the next tile, K first
        });
      }
      // fewer steps than copy instructions (head dims below the layout's): the rest of the copies follow here
      if constexpr (!I8 && kKS < 2 * kCopies)
        static_for<2 * kCopies - kKS>([&](auto C) { issue_copy(next, NEXT_BUF{}, std::integral_constant<int, kKS + decltype(C)::value>{}); });
    }
    // head_dim 256: the V^T fragments of the tile's first 16 keys set out now and arrive during the softmax
    const char* vb = &lds.v[buf][0];
    auto v_frags = [&](int step, uint4 (&af)[kTD]) __attribute__((always_inline)) {
#pragma unroll
      for (int td = 0; td < kTD; ++td) {
        const char* p0 = vb + v_off(td) + 16 * step * kRowB;
        const v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p0));
        const v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p0 + 8 * kRowB));
        af[td].x = __builtin_bit_cast(uint2, a0).x; af[td].y = __builtin_bit_cast(uint2, a0).y;
        af[td].z = __builtin_bit_cast(uint2, a1).x; af[td].w = __builtin_bit_cast(uint2, a1).y;
      }
    };
    uint4 afr[2][kTD];
    if constexpr (D == 256) {
      v_frags(0, afr[0]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- online softmax, one query row per lane (scores stay unscaled; the scale is folded
    //      into the exp2 argument) ----
    if constexpr (diag) {
      const int thr = min(cached + qrow, kv_len - 1) - j * kBN - 4 * hi;   // kv offset inside the tile must be <= thr
#pragma unroll
      for (int tk = 0; tk < NH; ++tk)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (32 * tk + 8 * (r >> 2) + (r & 3) > thr) s[tk][r] = -INFINITY;
    }
    // The chain starts from ordinary reads of one accumulator of each MFMA chain: the compiler keeps the
    // distance an MFMA result needs before a vector instruction may read it only for instructions it knows,
    // not for the v_max3 asm, and every max3 below depends on this first value (MFMAs finish in issue order,
    // so once the last instruction of a chain has delivered, the chain's other registers are final too).
    // Two chains, one per half, so that the dependent maxima are half as deep; both start from mx0.
    const float mx0 = fmaxf(s[0][15], s[NH - 1][15]);
    float mx = mx0;
    if constexpr (NH == 2) {
      float mx1 = mx0;
#pragma unroll
      for (int r = 0; r < 14; r += 2) {
        mx = max3(mx, s[0][r], s[0][r + 1]);
        mx1 = max3(mx1, s[1][r], s[1][r + 1]);
      }
      mx = max3(mx, s[0][14], s[1][14]);
      mx = fmaxf(mx, mx1);
    } else {
#pragma unroll
      for (int r = 0; r < 14; r += 2) mx = max3(mx, s[0][r], s[0][r + 1]);
      mx = fmaxf(mx, s[0][14]);
    }
    // the other half of the row's keys sits in lane l ^ 32: exchange on the vector unit (no LDS round trip, and
    // no wait behind the fragment reads queued there)
    mx = max_with_lane_xor32(mx);                      // tile maximum of the row, relative to the running one
    const bool grow = first || mx > 8.f;
    // head_dim 256: marked unlikely, so that the rescale sits out of line and the register allocator does not plan the
    // tile loop around it (for the other head dims the hint only moves blocks about: measured, no gain)
    if (D == 256 ? __builtin_expect(__any(grow), 0) : __any(grow)) {
      const float d = grow ? mx : 0.f;                 // the running maximum moves up by d (any finite d on the first tile)
      const float alpha = first ? 1.f : fast_exp2(-d); // nothing is accumulated yet on the first tile
      l *= alpha;
      if constexpr (D == 256) {
        // The accumulators live in the accumulator half of the register file, which only the matrix unit and these
        // moves reach: each is fetched, scaled and put back where it was, so the tile loop never holds a second copy
        // of all 128 in ordinary registers.  (Nothing is accumulated yet in a wave's first tile.)
        if (!first) {
#pragma unroll
        for (int td = 0; td < kTD; ++td)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float x = o[td][r];
            float t, y;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(x));
            t *= alpha;
            asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(y) : "v"(t));
            o[td][r] = y;
          }
        asm volatile("s_nop 7");                       // the moves' results are final before the matrix unit reads them
        }
      } else {
#pragma unroll
        for (int td = 0; td < kTD; ++td)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[td][r] *= alpha;
      }
      const float nm = neg_m[0] - d;
#pragma unroll
      for (int r = 0; r < 16; ++r) neg_m[r] = nm;
#pragma unroll
      for (int tk = 0; tk < NH; ++tk)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[tk][r] -= d;
      first = false;
    }
#pragma unroll
    for (int tk = 0; tk < NH; ++tk)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[tk][r] = fast_exp2(s[tk][r]);

    // ---- O^T += V^T P^T ----
    if constexpr (D == 256) {
      static_for<2 * NH>([&](auto STEP) {              // 16 kv rows per step; the next step's fragments set out first
        constexpr int step = decltype(STEP)::value, tk = step / 2, st = step % 2;
        uint4 pf;
        pf.x = pack2<T>(s[tk][8 * st + 0], s[tk][8 * st + 1]);
        pf.y = pack2<T>(s[tk][8 * st + 2], s[tk][8 * st + 3]);
        pf.z = pack2<T>(s[tk][8 * st + 4], s[tk][8 * st + 5]);
        pf.w = pack2<T>(s[tk][8 * st + 6], s[tk][8 * st + 7]);
        l = add_pair<T>(pf.w, add_pair<T>(pf.z, add_pair<T>(pf.y, add_pair<T>(pf.x, l))));
        if constexpr (step + 1 < 2 * NH) v_frags(step + 1, afr[(step + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(afr[step & 1][td], pf, o[td]);
      });
    } else {
      static_for<2 * NH>([&](auto STEP) {              // 16 kv rows per step
        constexpr int tk = decltype(STEP)::value / 2, st = decltype(STEP)::value % 2;
        uint4 pf;
        pf.x = pack2<T>(s[tk][8 * st + 0], s[tk][8 * st + 1]);
        pf.y = pack2<T>(s[tk][8 * st + 2], s[tk][8 * st + 3]);
        pf.z = pack2<T>(s[tk][8 * st + 4], s[tk][8 * st + 5]);
        pf.w = pack2<T>(s[tk][8 * st + 6], s[tk][8 * st + 7]);
        // row sum from the rounded weights, the ones the numerator uses; partial: this lane's kv rows only
        // (lanes l and l^32 are added at the end)
        l = add_pair<T>(pf.w, add_pair<T>(pf.z, add_pair<T>(pf.y, add_pair<T>(pf.x, l))));
        uint4 af[kTD];
        v_frags(decltype(STEP)::value, af);
#pragma unroll
        for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(af[td], pf, o[td]);
      });
    }
  };

  // Tile j lives in buffer j % 2.  The main loop is unrolled by two so that the buffer index is a compile-time
  // constant inside tile_step.  A wave's tiles are n_full complete ones and then those the causal diagonal runs
  // through: one when the rows start at a multiple of 32 keys (always, without a cached prefix), else up to two.
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using H1 = std::integral_constant<int, 1>;
  using H2 = std::integral_constant<int, 2>;
  auto full_step = [&](int j, auto BUF) {
    dma_wait_all();                    // this wave's share of tile j has landed
    __syncthreads();                   // ... and everybody else's; tile j-1 is no longer read
    tile_step(j, BUF, std::false_type{}, H2{}, j + 1 < ntiles);
  };
  auto diag_step = [&](int j, auto BUF) {
    dma_wait_all();
    __syncthreads();
    // no row of the wave reaches the second 32 keys of the tile: skip that half
    if (pos0 + kWaveRows - 1 < j * kBN + 32) tile_step(j, BUF, std::true_type{}, H1{}, j + 1 < ntiles);
    else tile_step(j, BUF, std::true_type{}, H2{}, j + 1 < ntiles);
  };
  int j = 0;
  if constexpr (I8) {
    // codes of tile j have landed and tile j - 1 is no longer read: send for tile j + 1, convert tile j
    auto stage = [&](int jj) {
      dma_wait_all();
      __syncthreads();
      const Scales sc_next = issue_codes(jj + 1, jj + 1 < ntiles);
      convert_tile(jj, sc_cur);
      sc_cur = sc_next;
      __syncthreads();                  // the 16-bit tile is complete
    };
    if (active) {
      for (; j < n_full; ++j) {
        stage(j);
        tile_step(j, B0{}, std::false_type{}, H2{}, false);
      }
      for (; j <= j_last; ++j) {
        stage(j);
        if (pos0 + kWaveRows - 1 < j * kBN + 32) tile_step(j, B0{}, std::true_type{}, H1{}, false);
        else tile_step(j, B0{}, std::true_type{}, H2{}, false);
      }
    }
    for (; j < ntiles; ++j) stage(j);
  }
  if (!I8 && active) {
    for (; j + 1 < n_full; j += 2) {
      full_step(j, B0{});
      full_step(j + 1, B1{});
    }
    if (j < n_full) {
      full_step(j, B0{});
      ++j;
    }
    for (; j <= j_last; ++j) {
      if (j & 1) diag_step(j, B1{});
      else diag_step(j, B0{});
    }
  }
  // Tiles that only other waves of the workgroup still compute on (their rows are further down): keep copying
  // this wave's share and meeting the barriers.  Kept out of the loop above so that the accumulators have one
  // straight-line life there.
  for (; !I8 && j < ntiles; ++j) {
    dma_wait_all();
    __syncthreads();
    if (j + 1 < ntiles) issue_tile(j + 1, (j + 1) & 1);
  }

  // ---- epilogue: normalise, transpose through LDS (the K buffers are free now), store whole rows ----
  // lane holds row l32, dims 32*td + 8*(r/4) + 4*hi + r%4  ->  wave-private [32 rows][256 B] tile with
  // 16-byte chunks xor-swizzled by row, read back as 16 B per lane so every global store is a full row.
  dma_wait_all();                                    // the zero fill issued during the last tile has landed
  __syncthreads();                                   // every wave is done reading K/V tiles
  if (!active) return;
  char* ot = &lds.k[0][0] + wave * (kWaveRows * kRowB);   // 4 waves x 32 rows = both K buffers
  {
    const float lt = l + __shfl_xor(l, 32, 64);
    const float inv = 1.f / lt;
    if (PAGED && a.lse != nullptr && hi == 0 && qrow < seq_len)
      a.lse[(int64_t)(seq_start + qrow) * a.num_heads + h] = __log2f(lt) - neg_m[0];
#pragma unroll
    for (int td = 0; td < kTD; ++td)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        uint2 w;
        w.x = pack2<T>(o[td][4 * r4 + 0] * inv, o[td][4 * r4 + 1] * inv);
        w.y = pack2<T>(o[td][4 * r4 + 2] * inv, o[td][4 * r4 + 3] * inv);
        *reinterpret_cast<uint2*>(ot + l32 * kRowB + (((4 * td + r4) ^ kswz(l32)) << 4) + 8 * hi) = w;
      }
  }
  // wave-private tile: the writes above and the reads below are ordered by the LDS queue of this wave
  T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
  for (int i = 0; i < kWaveRows / kCopyRows; ++i) {
    const int row = kCopyRows * i + lane / kChunks;
    const int c = lane % kChunks;
    const uint4 w = *reinterpret_cast<const uint4*>(ot + row * kRowB + ((c ^ kswz(row)) << 4));
    if (r0 + row < seq_len && c < DD / 8)
      store16_stream(out + ((int64_t)(seq_start + r0 + row) * a.num_heads + h) * DD + 8 * c, w);   // +2.5 % at config 2
  }
}

// D: the LDS layout (64, 128 or 256), DD: the data's head dimension.
template <typename T, bool PAGED, bool I8, int D, int DD>
static int launch_prefill_mfma_as(const PrefillArgs& a, hipStream_t stream) {
  const int group = a.num_heads / a.num_kv_heads;
  // query heads of a kv head per workgroup: 4 or 2 where they divide the group, else 1 (the workgroup is then four
  // row tiles of one head)
  const int hpw = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
  const int bm = kWaveRows * (kPfWaves / hpw);
  PrefillArgs b = a;
  // upper bound on the query tiles: every sequence may end with a partial tile; in the banded order (at most 64
  // sequences) every sequence may also end with a partial band of kBandRows / bm tiles
  b.band_shift = band_shift_for(a.total_tokens, a.num_seqs, bm, PAGED);
  b.tiles_x = a.num_seqs <= 64 ? (int)(a.total_tokens / bm + ((int64_t)a.num_seqs << b.band_shift))
                               : (int)(a.total_tokens / bm + a.num_seqs);
  b.heads_y = a.num_kv_heads * (group / hpw);
  b.band_bits = 1;
  while (((int64_t)1 << b.band_bits) <= a.total_tokens / (bm << b.band_shift) + 1) ++b.band_bits;
  const int64_t items = (int64_t)b.tiles_x * b.heads_y;
  const int64_t span = 8 * (int64_t)kXcdChunk;
  dim3 grid((unsigned)((items + span - 1) / span * span));
  const dim3 block(64 * kPfWaves);
  if (hpw == 4) prefill_mfma_kernel<T, 4, PAGED, D, I8, DD><<<grid, block, 0, stream>>>(b);
  else if (hpw == 2) prefill_mfma_kernel<T, 2, PAGED, D, I8, DD><<<grid, block, 0, stream>>>(b);
  else prefill_mfma_kernel<T, 1, PAGED, D, I8, DD><<<grid, block, 0, stream>>>(b);
  return launch_status();
}
template <typename T, bool PAGED, bool I8 = false>
static int launch_prefill_mfma(const PrefillArgs& a, hipStream_t stream) {
  return a.head_dim == 64 ? launch_prefill_mfma_as<T, PAGED, I8, 64, 64>(a, stream)
                          : launch_prefill_mfma_as<T, PAGED, I8, 128, 128>(a, stream);
}

// the paged form over a 16-bit cache, head_dim 64 or 128, bf16 / fp16 (prefill_varlen.hip)
int launch_prefill_paged_16bit(const PrefillArgs& a, int dtype, hipStream_t stream);
// the paged form over an INT8 cache (codes + fp32 scales), head_dim 64 or 128, bf16 / fp16 queries (prefill_varlen.hip)
int launch_prefill_paged_int8(const PrefillArgs& a, int dtype, hipStream_t stream);
// fp32 tensors, head_dim 128 or 64, packed or over a paged fp32 cache (prefill_f32.hip)
int launch_prefill_f32(const PrefillArgs& a, bool paged, hipStream_t stream);
// every other multiple of 8 from 32 to 120, and 256 (prefill_other_dims.hip, prefill_half_step_dims.hip); 16-bit element types only
bool prefill_mfma_other_dim(int head_dim);
int launch_prefill_mfma_other(const PrefillArgs& a, int dtype, bool paged, hipStream_t stream);

}  // namespace mvllm
