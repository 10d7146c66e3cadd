// Varlen causal flash-attention prefill for gfx950, two-group ("ping-pong") form.
// Replaces the Triton kernel of src/myvllm/layers/attention.py:111-209 for batches this kernel is built for
// (16-bit q/k/v, head_dim 128, an even number of query heads per kv head, at most 64 sequences); the launcher in
// prefill_varlen.hip falls back to prefill_mfma_kernel for everything else.
//
// One persistent workgroup of 8 waves per CU (two waves per SIMD, 160 KB of LDS).  A work item is one kv head, four
// of its query heads and a block of 64 consecutive query rows of one sequence; wave w owns query head w % 4 and the
// 32-row half w / 4 of the block.  (Where the heads per kv head are not a multiple of 4 an item is two heads and
// 128 rows: see pp_run.)  Waves 0-3 (group 0) and waves 4-7 (group 1) run the same tile loop one barrier
// interval apart: while one group feeds the matrix unit (O += V^T P^T of tile n, then S^T = K Q^T of tile n + 1: 32
// MFMAs, no other vector work) the other does the softmax of its tile on the vector unit, and they swap at every
// barrier.  The two waves that share a SIMD are then never both in their softmax nor both waiting for the matrix
// unit, which is what a workgroup per group (no ordering between them) left to chance.
//
// Everything a workgroup needs arrives in LDS by buffer_load ... lds: 64-row K and V tiles in rings of three,
// issued three barrier intervals before their first use, and each wave's 32 query rows, into a private 8 KB slot
// that is also the transposing buffer of the wave's output rows.  The tile stream runs on across item boundaries
// (the ring does not care which item a tile belongs to), the next item's Q rows are on their way while the current
// item is computed, and an item's output is normalised, transposed and stored during the softmax interval of the
// next item's first tile, so a workgroup pays the start-up latency once, not once per item.
//
// Items are dealt statically, heaviest first: level = index of the 64-row block inside its sequence (a block at
// level b walks b + 1 key tiles), levels descending, inside a level head slice then sequence.  The workgroups that
// share a list ("team": the workgroups of the XCDs that serve the same head slices, so that a kv head's keys stay in
// one L2) take ranks in serpentine order (r T + t in even rounds, r T + T - 1 - t in odd ones), which evens out the
// cost per workgroup.  Every wave finds its items from cu_seqlens with ballots; nothing is prepared by the host.
#include "prefill_tiles.h"

namespace mvllm {

namespace {

constexpr int kPpBN = 64;          // keys per tile
constexpr int kPpRing = 3;         // K and V tiles in flight
constexpr int kPpWaves = 8;
#ifndef MVLLM_PP_TIMELINE
#define MVLLM_PP_TIMELINE 0            // 1: the timing build of the probe library (per-tile clock stamps)
#endif


template <int D>
struct PpLds {
  static constexpr int kRowB = D * 2;
  static constexpr int kTileBytes = kPpBN * kRowB;
  static constexpr int kSlotBytes = 32 * kRowB;
  char k[kPpRing][kTileBytes];
  char v[kPpRing][kTileBytes];
  char qo[kPpWaves][kSlotBytes];    // per wave: Q rows of the next item on their way in, then the output rows on their way out
};

template <int N> __device__ __forceinline__ void vm_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// all waves of the workgroup; orders nothing but the compiler's own memory accesses (no LDS or memory counter is
// drained: data other waves read arrives by DMA, whose completion the issuing wave awaits explicitly)
__device__ __forceinline__ void pp_barrier() {
  __builtin_amdgcn_sched_barrier(0);            // no instruction of the softmax interval drifts into the matrix interval, nor back
  asm volatile("s_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// 16 bytes per lane to base + lane_off, streaming; lanes whose 16 bytes do not end inside `bytes` store nothing.
__device__ __forceinline__ void store16_buffer(void* base, uint32_t bytes, uint32_t lane_off, uint4 v) {
  const u32x4 w = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(w, __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)bytes, 0x00020000), (int)lane_off, 0, 2);
}

// 16 bytes per lane into LDS at m0_base + 16 * lane, from rsrc + lane_off.
__device__ __forceinline__ void dma16(v4i rsrc, uint32_t lane_off, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(lane_off), "s"(rsrc) : "m0", "memory");
}

}  // namespace

// One team's item list, walked in rank order.  Wave-uniform.
struct PpItems {
  int level;          // level the walk has reached (-1: past the last item)
  unsigned base;      // rank of that level's first item
};
struct PpItem {
  int seq_start, seq_len, rb;   // the sequence's query rows; the item's 64-row block of them
  int nt;             // index of the item's last key tile ( = rb without a cached prefix)
  int kvh, h0;        // kv head; first of the item's four query heads
  int seq, cached;    // paged mode: the sequence's row in the block table, its cached tokens
  bool valid;
};

// x / d for x < 2^16 by a multiplication: magic = 2^32 / d + 1 (d > 1; d == 1 has magic 0 and is passed through).
__device__ __forceinline__ unsigned div_small(unsigned x, unsigned d, unsigned magic) {
  return d == 1u ? x : __umulhi(x, magic);
}

// PAGED: prefill of the tokens that follow a cached prefix.  Query row r of a sequence sits at key position c + r
// (c = its cached tokens); every key, cached or new, is read from the paged cache through the block table (the store
// precedes this call), 16 rows = one piece of one block per wave and tile.  An item's key tiles are 0 ..
// ceil(c / 64) + rb, and unless c is a multiple of 64 the causal diagonal crosses the last two of them.
//
// HPI: query heads per item.  4: the item is a 64-row block, wave w has head w % 4 and rows 32 GRP ...  2 (two or six
// ... query heads per kv head): the item is a 128-row block of two heads, wave w has head w % 2 and rows
// 64 GRP + 32 ((w % 4) / 2) ...; the block's last key tile is then the index of its second 64-row step, the
// diagonal crosses its last two tiles (three over a prefix in general position), and the waves of its first 64 rows
// compute a last tile they see nothing of.
template <typename T, int D, int GRP, bool PAGED, int HPI>
__device__ __forceinline__ void pp_run(const PrefillPpArgs& a, PpLds<D>& lds, const int wave) {
  static_assert(HPI == 4 || HPI == 2, "items of four or of two query heads");
  constexpr int kTPB = 4 / HPI;                // 64-row steps (and diagonal key tiles) per item
  constexpr int kRPI = 64 * kTPB;              // query rows per item
  constexpr int kRowB = D * 2;
  constexpr int kTileBytes = kPpBN * kRowB;
  constexpr int kKS = D / 16;
  constexpr int kTD = D / 32;
  static_assert(D == 128, "swizzles and copy shapes are written for 256-byte rows");
  auto kswz = [](int row) __attribute__((always_inline)) { return row & 15; };
  auto vswz = [](int row) __attribute__((always_inline)) { return ((row & 3) << 2) | (row & 1); };

  const int lane = threadIdx.x & 63;
  const int l32 = lane & 31;
  const int hi = lane >> 5;
  const int wq = wave & 3;                     // wave inside its group: its piece of the group's copies
  const int wh = wq & (HPI - 1);               // query head inside the item
  const int row_off = 32 * kTPB * GRP + 32 * (wq / HPI);   // the wave's 32 query rows inside the item's block

#if MVLLM_PP_TIMELINE
  // Timing build (the probe library): the waves of one workgroup log the shader clock at the four corners of every
  // tile (softmax begins, softmax done, matrix part begins, matrix part done), `timeline_entries` stamps per wave.
  // A stamp costs about a hundred clocks, so the logged intervals are each that much longer than in the product build.
  unsigned long long* tlog = a.timeline + (size_t)wave * a.timeline_entries;
  int tn = 0;
  const bool tlogging = MVLLM_PP_TIMELINE == 1 && a.timeline != nullptr && (int)blockIdx.x == a.timeline_block;
  // timeline_block < 0: instead, wave 4 of every workgroup logs when it began and ended and how many items and tiles
  // it went through, four entries per workgroup.
  const unsigned long long t_begin = __builtin_amdgcn_s_memtime();
  int t_items = 0, t_tiles = 0;
#define TCOUNT(items, tiles) do { t_items += (items); t_tiles += (tiles); } while (0)
#define TSTAMP() do { if (MVLLM_PP_TIMELINE == 1 && tlogging && tn < a.timeline_entries) { const unsigned long long t_ = __builtin_amdgcn_s_memtime(); if (lane == 0) tlog[tn] = t_; ++tn; } } while (0)
#else
#define TSTAMP() do {} while (0)
#define TCOUNT(items, tiles) do {} while (0)
#endif
  // ---- the batch, one sequence per lane ----
  int lo = 0, len = 0, cached = 0, kv_len = 0;
  if (lane < a.num_seqs) {
    lo = a.cu_seqlens[lane];
    len = a.cu_seqlens[lane + 1] - lo;
    if (PAGED) {
      kv_len = a.cu_seqlens_k[lane + 1] - a.cu_seqlens_k[lane];
      cached = kv_len > len ? kv_len - len : 0;
    }
  }
  const int nb = (len + kRPI - 1) / kRPI;      // item blocks of the lane's sequence
  // An item's level is the index of its last key tile: block rb of a sequence with c cached tokens has level
  // (c + kRPI - 1) / 64 + kTPB rb, so the lane's sequence owns every kTPB-th level from lvl0 to lvl_end - 1.
  const int lvl0 = (cached + kRPI - 1) >> 6;
  const int lvl_end = nb > 0 ? lvl0 + kTPB * (nb - 1) + 1 : 0;
  int top = 0;                                 // one past the highest level in the batch
  for (int bit = a.level_bits - 1; bit >= 0; --bit) {
    const int trial = top | (1 << bit);
    if (__ballot(lvl_end >= trial) != 0ull) top = trial;
  }

  // ---- which items are this workgroup's ----
  const unsigned wg = blockIdx.x;
  const unsigned xcd = wg & 7u;
  const int team = (int)(xcd % (unsigned)a.n_teams);
  const unsigned TS = (unsigned)a.team_size;
  const unsigned t = (wg >> 3) * (8u / (unsigned)a.n_teams) + xcd / (unsigned)a.n_teams;   // index inside the team
  const unsigned spt = (unsigned)(a.slices / a.n_teams);                                  // slices per team
  const int group = a.num_heads / a.num_kv_heads;
  const int chunks = group / HPI;
  // The workgroup's k-th item is rank k TS + (t or, in odd rounds, TS - 1 - t) of the team's list.  Locating an item
  // costs a hundred-odd instructions per wave, and two cursors go through the same items (the copies run ahead of the
  // arithmetic), so every item is located once and kept in lane (k mod 16) of four registers until both have passed.
  // Ranks are dealt in rounds of TS, forwards and backwards in turn; the serpentine leaves the team's first
  // workgroups the most tiles (the first rounds, whose costs fall fastest, weigh most), so a last round that is not
  // full always runs backwards: its items, each worth three to four tiles of fixed cost, go to the workgroups that
  // have the least.
  int team_items = nb;
#pragma unroll
  for (int step = 1; step < 64; step <<= 1) team_items += __shfl_xor(team_items, step, 64);
  team_items = __builtin_amdgcn_readfirstlane(team_items) * (int)spt;
  const unsigned short_round = (unsigned)team_items % TS != 0u ? (unsigned)team_items / TS : 0xffffffffu;
  PpItems walk = {top - 1, 0u};
  int produced = 0;
  int kept_start = 0, kept_len = 0, kept_rb = 0, kept_heads = 0, kept_seq = 0;   // kept_rb: the level; kept_seq: paged only
  auto produce = [&]() {
    const unsigned round = (unsigned)produced;
    const bool backwards = (round & 1u) != 0u || round == short_round;
    const unsigned R = round * TS + (backwards ? TS - 1u - t : t);
    unsigned long long mask = 0ull;
    unsigned cnt = 0;
    while (walk.level >= 0) {
      mask = __ballot(walk.level < lvl_end && walk.level >= lvl0 && (kTPB == 1 || ((walk.level - lvl0) & (kTPB - 1)) == 0));
      cnt = (unsigned)__popcll(mask);
      const unsigned items = cnt * spt;
      if (R - walk.base < items) break;
      walk.base += items;
      --walk.level;
    }
    int seq_start = 0, seq_len = 0, heads = 0, seq = 0;
    if (walk.level >= 0) {
      // inside a level: sequence-major, the team's slices of one sequence side by side
      const unsigned idx = R - walk.base;
      const unsigned qth = div_small(idx, spt, a.spt_magic);
      const unsigned sl = idx - qth * spt;
      const int below = __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
      const unsigned long long pick = __ballot(((mask >> lane) & 1ull) != 0ull && below == (int)qth);
      const int owner = __ffsll((long long)pick) - 1;
      seq_start = __builtin_amdgcn_readlane(lo, owner);
      seq_len = __builtin_amdgcn_readlane(len, owner);
      seq = owner;
      const unsigned y = (unsigned)team + (unsigned)a.n_teams * sl;
      const unsigned kvh = div_small(y, (unsigned)chunks, a.chunks_magic);
      heads = (int)((kvh << 16) | (kvh * (unsigned)group + (y - kvh * (unsigned)chunks) * (unsigned)HPI));
    }
    const int at = produced & 15;
    kept_start = lane == at ? seq_start : kept_start;
    kept_len = lane == at ? seq_len : kept_len;
    kept_rb = lane == at ? walk.level : kept_rb;     // -1: no such item
    kept_heads = lane == at ? heads : kept_heads;
    if (PAGED) kept_seq = lane == at ? seq : kept_seq;
    ++produced;
  };
  auto item_at = [&](int k) {
    while (produced <= k) produce();
    PpItem it;
    const int at = k & 15;
    it.seq_start = __builtin_amdgcn_readlane(kept_start, at);
    it.seq_len = __builtin_amdgcn_readlane(kept_len, at);
    it.nt = __builtin_amdgcn_readlane(kept_rb, at);
    const int heads = __builtin_amdgcn_readlane(kept_heads, at);
    it.kvh = (int)((unsigned)heads >> 16);
    it.h0 = heads & 0xffff;
    it.valid = it.nt >= 0;
    it.seq = 0; it.cached = 0;
    if (PAGED) {
      it.seq = __builtin_amdgcn_readlane(kept_seq, at);
      it.cached = __builtin_amdgcn_readlane(cached, it.seq);
    }
    it.rb = (it.nt - ((it.cached + kRPI - 1) >> 6)) / kTPB;
    return it;
  };

  int ci = 0;                                  // items handed to the arithmetic so far
  PpItem cur = item_at(ci++);
  if (!cur.valid) return;                      // no item for this workgroup (all waves agree)
  PpItem nxt = item_at(ci++);
  int di = 0;
  PpItem dit = cur;                            // item the copy cursor is in
  int dj = 0;                                  // ... and its tile there

  const T* qg = reinterpret_cast<const T*>(a.q);
  const char* kg = reinterpret_cast<const char*>(a.k);
  const char* vg = reinterpret_cast<const char*>(a.v);
  const int kv_row_bytes = a.num_kv_heads * kRowB;
  const int q_row_bytes = a.num_heads * kRowB;
  const int total_rows = (int)a.total_tokens;

  // ---- copies ----
  // Group 0 copies the K tiles, group 1 the V tiles, each at the start of its softmax interval: wave w of a group
  // moves rows 16 w .. 16 w + 15 of the tile, 4 rows (1 KB) per instruction.  A copy is issued three barrier
  // intervals before the barrier that publishes it and overwrites the tile three places back in its ring, whose
  // last readers finished an interval before.
  const int ld_row = lane >> 4, ld_chunk = lane & 15;
  uint32_t src_off[4];                         // (paged: relative to the wave's own piece of the tile)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 16 * wq + 4 * i + ld_row;
    src_off[i] = (uint32_t)((PAGED ? row - 16 * wq : row) * kv_row_bytes + ((ld_chunk ^ (GRP == 0 ? kswz(row) : vswz(row))) << 4));
  }
  const char* copy_src = GRP == 0 ? kg : vg;
  const uint32_t lds_copy0 = (GRP == 0 ? lds_address(&lds.k[0][0]) : lds_address(&lds.v[0][0])) + (uint32_t)(16 * wq * kRowB);
  // A tile's descriptor starts at its first row (for the item's kv head) and ends with the tensor, so rows past the
  // last token arrive as zeros; size 0 (nothing read, zeros written) when the stream has ended.  The cursor keeps
  // the tile's byte offset and the rows that follow it.
  const int rows_4g = (int)(0xffffffffu / (uint32_t)kv_row_bytes);
  int64_t d_off = 0;                           // byte offset of the cursor's tile in k (and v)
  int d_rows_left = 0;                         // rows from the tile's first to the tensor's last; <= 0: no tile
  int d_head_off = 0;                          // byte offset of the kv head inside a row
  // Paged: the wave's 16 rows of the cursor's tile are one piece of one cache block (block_size % 16 == 0).  Its
  // table entry is fetched with a scalar load one copy step ahead (`d_phys`), so that no step waits for it; the
  // descriptor starts at the piece and ends with the sequence's last key, so rows that were never written, unmapped
  // blocks and tiles past the stream's end arrive as zeros.
  int d_phys = -1;                             // table entry of the cursor's piece
  int d_in_off = 0;                            // ... and the byte offset of its first row (at the item's kv head) inside that block
  int d_kv_len = 0;                            // keys of the cursor's sequence
  auto fetch_entry = [&]() {                   // for the cursor's tile (dit, dj)
    if constexpr (PAGED) {
      const unsigned pos = (unsigned)(kPpBN * dj + 16 * wq);
      const unsigned bi = div_small(pos, (unsigned)a.block_size, a.block_magic);
      d_in_off = (int)(pos - bi * (unsigned)a.block_size) * kv_row_bytes + d_head_off;
      // (read through the constant address space: a scalar load, which the copies' vmcnt accounting does not see; a
      // vector load here would make the compiler wait for every copy in flight before each use of the entry)
      typedef const __attribute__((address_space(4))) int32_t* ConstTable;
      const ConstTable table = reinterpret_cast<ConstTable>(reinterpret_cast<uintptr_t>(a.block_tables));
      const int64_t at = (int64_t)__builtin_amdgcn_readfirstlane(dit.seq) * a.max_num_blocks + __builtin_amdgcn_readfirstlane((int)bi);
      d_phys = dit.valid && (int)bi < a.max_num_blocks ? table[at] : -1;
    }
  };
  auto enter_item = [&]() {                    // the cursor's tile = first tile of `dit`
    d_head_off = dit.kvh * kRowB;
    if constexpr (PAGED) {
      d_kv_len = dit.valid ? __builtin_amdgcn_readlane(kv_len, dit.seq) : 0;
    } else {
      d_off = (int64_t)dit.seq_start * kv_row_bytes + d_head_off;
      d_rows_left = dit.valid ? total_rows - dit.seq_start : 0;
    }
  };
  enter_item();
  fetch_entry();
  int d_slot = 0;                              // ring slot of the cursor's tile ( = its stream index % 3)
  auto issue_copy = [&]() {                    // the cursor's tile -> its ring slot
    v4i r;
    if constexpr (PAGED) {
      const int pos = kPpBN * dj + 16 * wq;
      const int valid = d_kv_len - pos < 16 ? d_kv_len - pos : 16;
      const bool ok = dit.valid && valid > 0 && (unsigned)d_phys < (unsigned)a.num_blocks32;   // (-1: not mapped)
      const uint32_t size = ok ? (uint32_t)(valid - 1) * (uint32_t)kv_row_bytes + (uint32_t)kRowB : 0u;
      const int64_t start = ok ? (int64_t)d_phys * a.block_bytes + d_in_off : 0;
      r = make_rsrc(copy_src + start, size);
    } else {
      const uint32_t size = d_rows_left <= 0        ? 0u
                            : d_rows_left > rows_4g ? 0xffffffffu
                                                    : (uint32_t)d_rows_left * (uint32_t)kv_row_bytes - (uint32_t)d_head_off;
      r = make_rsrc(copy_src + d_off, size);
    }
    const uint32_t dst = lds_copy0 + (uint32_t)(d_slot * kTileBytes);
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(r, src_off[i], dst + 1024u * i);
    d_slot = d_slot == kPpRing - 1 ? 0 : d_slot + 1;
  };
  auto copy_step = [&]() {
    issue_copy();
    if (dit.valid) {
      if (++dj > dit.nt) {
        dit = item_at(++di);
        dj = 0;
        enter_item();
      } else if constexpr (!PAGED) {
        d_off += (int64_t)kPpBN * kv_row_bytes;      // the next 64 rows of the same sequence and head
        d_rows_left -= kPpBN;
      }
      fetch_entry();
    }
  };
  // The same where the caller knows that the cursor stays inside its item (the cursor is two tiles ahead of the
  // arithmetic, so this holds in tiles 1 .. nt - 3 of an item): no test, no item located, and none of the register
  // copies that the merge with that path costs in every tile.
  auto copy_step_inside = [&]() {
    issue_copy();
    ++dj;
    if constexpr (!PAGED) {
      d_off += (int64_t)kPpBN * kv_row_bytes;
      d_rows_left -= kPpBN;
    }
    fetch_entry();
  };
  // Q rows of an item -> this wave's slot, 4 rows per instruction, chunks swizzled like a K tile's
  const uint32_t lds_q = lds_address(&lds.qo[wave][0]);
  auto copy_q = [&](const PpItem& it) {
    const int h = it.h0 + wh;
    const int row = it.seq_start + it.rb * kRPI + row_off;
    const int rows_left = total_rows - row;
    const int rows_4g = (int)(0xffffffffu / (uint32_t)q_row_bytes);
    const uint32_t size = rows_left <= 0 ? 0u
                          : rows_left > rows_4g ? 0xffffffffu
                                                : (uint32_t)rows_left * (uint32_t)q_row_bytes - (uint32_t)(h * kRowB);
    const v4i r = make_rsrc(reinterpret_cast<const char*>(qg) + (int64_t)row * q_row_bytes + (int64_t)h * kRowB, size);
    int lane_q = lane;
    asm volatile("" : "+v"(lane_q));              // the eight source offsets are computed per item, not kept in registers
    const int qrow = lane_q >> 4, qchunk = lane_q & 15;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int rowi = 4 * i + qrow;
      const uint32_t off = (uint32_t)(rowi * q_row_bytes + ((qchunk ^ kswz(rowi)) << 4));
      dma16(r, off, lds_q + (uint32_t)(i * 1024));
    }
  };

  // ---- per-lane LDS offsets of the operand fragments (as in prefill_mfma_kernel) ----
  const int i16 = lane & 15;
  const int half = (lane >> 4) & 1;
  int k_off[kKS];
#pragma unroll
  for (int ks = 0; ks < kKS; ++ks) k_off[ks] = l32 * kRowB + (((2 * ks + hi) ^ kswz(l32)) << 4);
  const int v_row = 4 * hi + (i16 >> 2);
  int v_off[kTD];
#pragma unroll
  for (int td = 0; td < kTD; ++td)
    v_off[td] = v_row * kRowB + (((4 * td + 2 * half + ((i16 & 3) >> 1)) ^ vswz(v_row)) << 4) + ((i16 & 1) << 3);

  // ---- state ----
  uint4 qf[kKS];
  v16f o[kTD];
  v16f s[2];
  uint4 pf[4];                                  // P of the tile whose softmax was last, packed: [2 tk + st]
  float l = 0.f;
  // Running maximum of the lane's row, negated, in all 16 registers of an accumulator tuple: the score products
  // start from it (C operand of their first MFMA), so a tile's scores arrive as  score * scale * log2 e - m, ready
  // for exp2.  (An item's first tile starts from zero instead: its maximum is not known yet.)
  v16f neg_m;
#pragma unroll
  for (int r = 0; r < 16; ++r) neg_m[r] = 0.f;
#pragma unroll
  for (int td = 0; td < kTD; ++td)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[td][r] = 0.f;

  // slot -> registers, times scale * log2 e (rounded to the element type once), so that the scores leave the matrix
  // unit as exp2 arguments.  The multiplications run in a matrix interval, whose wave has vector slots to spare.
  auto read_q = [&]() {
    const char* qs = &lds.qo[wave][0];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) qf[ks] = *reinterpret_cast<const uint4*>(qs + k_off[ks]);
  };
  auto scale_q = [&](auto QUARTER) {              // a quarter of the fragments
#pragma unroll
    for (int ks = 2 * decltype(QUARTER)::value; ks < 2 * decltype(QUARTER)::value + 2; ++ks) {
      qf[ks].x = scale_pair<T>(qf[ks].x, a.scale_log2);
      qf[ks].y = scale_pair<T>(qf[ks].y, a.scale_log2);
      qf[ks].z = scale_pair<T>(qf[ks].z, a.scale_log2);
      qf[ks].w = scale_pair<T>(qf[ks].w, a.scale_log2);
    }
  };
  auto load_q = [&]() {
    read_q();
    static_for<4>([&](auto QUARTER) { scale_q(QUARTER); });
  };
  // Operand fragments from LDS.  K: rows l32 and l32 + 32 of the tile in K ring slot `slot`, dims 16 ks + 8 hi ..;
  // V^T: the transposing reads of the 16 keys of `step` ( = 2 tk + st) of the tile in V ring slot `slot`.
  auto k_frags = [&](int slot, auto KS, uint4 (&kf)[2]) {
    constexpr int ks = decltype(KS)::value;
    const char* kb = &lds.k[0][0] + slot * kTileBytes + k_off[ks];
    kf[0] = *reinterpret_cast<const uint4*>(kb);
    kf[1] = *reinterpret_cast<const uint4*>(kb + 32 * kRowB);
  };
  auto v_frags = [&](int slot, auto STEP, uint4 (&af)[kTD]) {
    constexpr int step = decltype(STEP)::value;
    const char* vb = &lds.v[0][0] + slot * kTileBytes + 16 * step * kRowB;
#pragma unroll
    for (int td = 0; td < kTD; ++td) {
      const char* p0 = vb + v_off[td];
      const v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p0));
      const v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p0 + 8 * kRowB));
      af[td].x = __builtin_bit_cast(uint2, a0).x; af[td].y = __builtin_bit_cast(uint2, a0).y;
      af[td].z = __builtin_bit_cast(uint2, a1).x; af[td].w = __builtin_bit_cast(uint2, a1).y;
    }
  };
  // the scores of the stream's first tile (the later ones are computed at the end of each matrix interval)
  auto first_scores = [&](int slot) {
    static_for<kKS>([&](auto KS) {
      constexpr int ks = decltype(KS)::value;
      uint4 kf[2];
      k_frags(slot, KS, kf);
      if constexpr (ks == 0) {
        v16f z;
#pragma unroll
        for (int r = 0; r < 16; ++r) z[r] = 0.f;
#pragma unroll
        for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf[tk], qf[0], z);
      } else {
#pragma unroll
        for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf[tk], qf[ks], s[tk]);
      }
    });
  };
  // An item's output leaves in two steps.  stage_out, in the matrix interval of the item's last tile (once the next
  // item's Q rows have been read out of the slot): O^T / row sum, rounded, into the wave's slot, transposed.
  // write_out, in the next softmax interval: whole rows from the slot to memory (rows past the sequence's end are not
  // stored).
  T* out = reinterpret_cast<T*>(a.out);
  auto stage_out = [&](auto TD, float inv) {     // 32 of the 128 dims
    constexpr int td = decltype(TD)::value;
    char* orow = &lds.qo[wave][0] + l32 * kRowB + 8 * hi;
    const int oswz = kswz(l32);
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
        uint2 w;
        w.x = pack2<T>(o[td][4 * r4 + 0] * inv, o[td][4 * r4 + 1] * inv);
        w.y = pack2<T>(o[td][4 * r4 + 2] * inv, o[td][4 * r4 + 3] * inv);
        *reinterpret_cast<uint2*>(orow + (((4 * td + r4) ^ oswz) << 4)) = w;
      }
  };
  auto write_out = [&](int seq_start, int seq_len, int rb, int h0) {
    const char* ot = &lds.qo[wave][0];
    int lane_o = lane;
    asm volatile("" : "+v"(lane_o));
    const int orow = lane_o >> 4, ochunk = lane_o & 15;
    const int r0 = rb * kRPI + row_off;
    // The descriptor ends with the head's part of the sequence's last row, so the stores of rows past it are dropped
    // by the bounds check: all eight are always issued, as the wait counts assume.
    const int rows = seq_len - r0 < 32 ? seq_len - r0 : 32;
    const uint32_t size = rows > 0 ? (uint32_t)(rows - 1) * (uint32_t)q_row_bytes + (uint32_t)kRowB : 0u;
    char* base = reinterpret_cast<char*>(out) + (int64_t)(seq_start + r0) * q_row_bytes + (int64_t)(h0 + wh) * kRowB;
    const uint32_t off0 = (uint32_t)(orow * q_row_bytes + 16 * ochunk);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 4 * i + orow;
      const uint4 w = *reinterpret_cast<const uint4*>(ot + row * kRowB + ((ochunk ^ kswz(row)) << 4));
      store16_buffer(base, size, off0 + (uint32_t)(4 * i) * (uint32_t)q_row_bytes, w);
    }
  };
  // The barrier that ends a softmax interval publishes the copy step issued in the wave's previous softmax interval:
  // everything but the `later` vector memory instructions issued in this one (its copy step and, in an item's first
  // tile, the previous item's 8 output stores and the next item's 8 Q copies: the bounds-checked stores are issued
  // whatever the sequence's length, so the count is exact) must have completed.  (Letting the previous interval's
  // stores and Q copies stay in flight as well was measured and is slower.)
  auto wait_copies = [&](int later) {
    if (later == 4) vm_wait<4>();
    else if (later == 12) vm_wait<12>();
    else if (later == 20) vm_wait<20>();
    else vm_wait<0>();
  };

  // ---- start: the first item's Q rows and the first three copy steps ----
  copy_q(cur);
  copy_step();
  copy_step();
  vm_wait<0>();
  pp_barrier();
  load_q();
  int c_slot = 0;                               // ring slot of the tile whose softmax comes next
  int p_seq_start = 0, p_seq_len = 0, p_rb = 0, p_h0 = 0;   // item whose output waits in the slot
  bool have_prev = false;

  if (GRP == 1) pp_barrier();                   // group 1 runs one interval behind
  first_scores(c_slot);
  asm volatile("" : "+v"(s[0]), "+v"(s[1]));
  pp_barrier();

  // The causal diagonal runs through half GRP of an item's last tile: key offset 8 (r / 4) + r % 4 + 4 hi inside
  // that half against query row l32.  Group 0's rows see nothing of the second half, group 1's all of the first.
  auto mask_diagonal = [&]() {
    int lim = l32 - 4 * hi;
    asm volatile("" : "+v"(lim));                 // computed here, not kept as sixteen lane masks across the loop
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if (8 * (r >> 2) + (r & 3) > lim) s[GRP][r] = -INFINITY;
      if (GRP == 0) s[1][r] = -INFINITY;
    }
  };
  // The diagonal against tile j of `cur` in general position (over a cached prefix; items of two heads).  Query row
  // l32 of this wave sits at key position cached + kRPI rb + row_off + l32; the lane's keys in the tile are
  // 64 j + 32 tk + 8 (r / 4) + r % 4 + 4 hi.  A wave whose rows all lie above the tile masks all of it: its weights
  // are zeros then, and the running maximum, which only a large row sum moves, stays.
  auto mask_tile = [&](int j) {
    int lim = cur.cached + kPpBN * (kTPB * cur.rb - j) + row_off + l32 - 4 * hi;
    asm volatile("" : "+v"(lim));
#pragma unroll
    for (int tk = 0; tk < 2; ++tk)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * tk + 8 * (r >> 2) + (r & 3) > lim) s[tk][r] = -INFINITY;
  };
  auto tile_max = [&]() {                        // maximum of the lane's row over the tile, relative to the running one
    const float mx0 = fmaxf(s[0][15], s[1][15]);
    float mx = mx0, mx1 = mx0;
#pragma unroll
    for (int r = 0; r < 14; r += 2) {
      mx = max3(mx, s[0][r], s[0][r + 1]);
      mx1 = max3(mx1, s[1][r], s[1][r + 1]);
    }
    mx = max3(mx, s[0][14], s[1][14]);
    mx = fmaxf(mx, mx1);
    return max_with_lane_xor32(mx);
  };
  // P = exp2(s - d) packed into pf (s itself is kept: a tile whose weights turn out too large is redone from it);
  // returns the lane's share of the row sum (of the weights before they are rounded to 16 bits: the roundings are
  // unbiased and average out over a row).  SHIFT: d != 0.
  auto weights = [&](auto SHIFT, float d) {
    float sum = 0.f;
#pragma unroll
    for (int tk = 0; tk < 2; ++tk)
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        float e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float x = s[tk][8 * st + i];
          e[i] = fast_exp2(decltype(SHIFT)::value ? x - d : x);
        }
        uint4 p;
        p.x = pack2<T>(e[0], e[1]);
        p.y = pack2<T>(e[2], e[3]);
        p.z = pack2<T>(e[4], e[5]);
        p.w = pack2<T>(e[6], e[7]);
        // Row sum with ordinary additions, four short chains.  (v_dot2_f32_bf16 on the packed pairs would halve the
        // instruction count, but the dot instructions queue behind the other group's MFMAs: sixteen of them took as
        // long as a whole matrix interval.)
        sum += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
        pf[2 * tk + st] = p;
      }
    return sum;
  };
  auto set_neg_m = [&](float v) {
#pragma unroll
    for (int r = 0; r < 16; ++r) neg_m[r] = v;
  };
  // The matrix interval after the softmax of tile j of `cur`: O^T (+)= V^T P^T of that tile (FRESH: from zero, the
  // item's first tile), then S^T = K Q^T of the stream's next tile, which belongs to the next item when j is the
  // item's last (its Q rows were copied during this item's first softmax interval).  32 MFMAs in eight stages of
  // four; every operand fragment is requested two stages (8 MFMAs, 256 matrix-unit clocks) before the stage that
  // uses it, because nothing else runs on this SIMD's matrix unit meanwhile that could cover an LDS round trip.
  // vf0, vf1: the V^T fragments of the tile's first two steps, requested before the barrier.  Group 0 also issues
  // its share of the next copy step here, one instruction per stage.  Returns false when the stream ends here.
  // A wave issues about one instruction in five clocks, an MFMA keeps the matrix unit for 32: at most five other
  // instructions fit between two MFMAs without a bubble, so each stage's fragment reads and their address
  // arithmetic are dealt out between its four MFMAs instead of standing in front of them.
  auto stage_end = [&](int reads_per_mfma, int others_per_mfma) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                   // one MFMA
      if (reads_per_mfma == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // LDS reads
      else if (reads_per_mfma == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      // vector instructions (a fragment's address; in an item's last tile the Q scaling and the output's
      // normalisation) and the output's LDS writes
      if (others_per_mfma == 1) __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);
      else if (others_per_mfma == 8) {
        __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // The compiler computes a value where it is first used, and moves pure arithmetic across a barrier freely.  These
  // empty statements make the softmax's results exist before the barrier that ends its interval, and the matrix
  // interval's before the one that ends it, so that each interval holds the work it is named for.
  auto pin_weights = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(pf[i].x), "+v"(pf[i].y), "+v"(pf[i].z), "+v"(pf[i].w));
    asm volatile("" : "+v"(l), "+v"(neg_m));
  };
  auto pin_products = [&]() {
    asm volatile("" : "+v"(s[0]), "+v"(s[1]));
    asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
  };
  // LAST (compile time: an item's last tile has a code path of its own, so the others carry none of its branches):
  // the next item's Q rows are read out of the slot after the P V MFMAs; their scaling, and the normalisation of the
  // item's output and its way into the slot, are dealt out between the K Q^T MFMAs of the next item's first tile.  When the stream ends here both still run, on whatever the slot and the next ring
  // tile hold, and nothing uses the results.
  auto matrix_interval = [&](auto FRESH, auto LAST, bool single, uint4 (&vf0)[kTD], uint4 (&vf1)[kTD]) {
    using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>; using I5 = std::integral_constant<int, 5>;
    using I6 = std::integral_constant<int, 6>; using I7 = std::integral_constant<int, 7>;
    constexpr bool kFresh = decltype(FRESH)::value, kLast = decltype(LAST)::value;
    static_assert(!(kFresh && kLast), "an item's first tile finds out at run time whether it is also the last");
    const bool last = kFresh ? single : kLast;
    const int n_slot = c_slot == kPpRing - 1 ? 0 : c_slot + 1;
    const bool more = !last || nxt.valid;
    // this wave's MFMAs go in front of the other group's vector instructions on the shared SIMD
    __builtin_amdgcn_s_setprio(3);
    uint4 vf2[kTD], vf3[kTD];
    uint4 kf0[2], kf1[2], kf2[2], kf3[2], kf4[2], kf5[2], kf6[2], kf7[2];
    // stage A
    v_frags(c_slot, I2{}, vf2);
    if constexpr (kFresh) {
      v16f z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
#pragma unroll
      for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(vf0[td], pf[0], z);
    } else {
#pragma unroll
      for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(vf0[td], pf[0], o[td]);
    }
    stage_end(2, 1);
    // stage B
    v_frags(c_slot, I3{}, vf3);
#pragma unroll
    for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(vf1[td], pf[1], o[td]);
    stage_end(2, 1);
    // stage C
    k_frags(n_slot, I0{}, kf0); k_frags(n_slot, I1{}, kf1);      // (read and not used when the stream ends here)
#pragma unroll
    for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(vf2[td], pf[2], o[td]);
    stage_end(1, 1);
    // stage D
    k_frags(n_slot, I2{}, kf2); k_frags(n_slot, I3{}, kf3);
#pragma unroll
    for (int td = 0; td < kTD; ++td) o[td] = mfma32x32x16<T>(vf3[td], pf[3], o[td]);
    stage_end(1, 1);
    float inv = 0.f;
    if constexpr (kFresh) {
      if (last) {                                // a single tile: no other work to hide these behind
        vm_wait<0>();
        load_q();
        inv = __builtin_amdgcn_rcpf(sum_with_lane_xor32(l));
        static_for<4>([&](auto TD) { stage_out(TD, inv); });
      }
    }
    if constexpr (kLast) {
      // the next item's Q rows, copied since this item's first softmax interval; one copy step was issued behind
      // them
      vm_wait<4>();
      read_q();
      inv = __builtin_amdgcn_rcpf(sum_with_lane_xor32(l));
      scale_q(I0{});
      __builtin_amdgcn_sched_barrier(0);
    }
    // stage E
    k_frags(n_slot, I4{}, kf4); k_frags(n_slot, I5{}, kf5);
    if (last) {
      // another item's first tile: its maximum is not known yet, the scores arrive as they are
      v16f z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
#pragma unroll
      for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf0[tk], qf[0], z);
    } else {
#pragma unroll
      for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf0[tk], qf[0], neg_m);
    }
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf1[tk], qf[1], s[tk]);
    if constexpr (kLast) { scale_q(I1{}); stage_out(I0{}, inv); }
    stage_end(1, kLast ? 8 : 1);
    // stage F
    k_frags(n_slot, I6{}, kf6); k_frags(n_slot, I7{}, kf7);
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf2[tk], qf[2], s[tk]);
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf3[tk], qf[3], s[tk]);
    if constexpr (kLast) { scale_q(I2{}); stage_out(I1{}, inv); }
    stage_end(1, kLast ? 8 : 1);
    // stage G
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf4[tk], qf[4], s[tk]);
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf5[tk], qf[5], s[tk]);
    if constexpr (kLast) { scale_q(I3{}); stage_out(I2{}, inv); }
    stage_end(0, kLast ? 8 : 0);
    // stage H
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf6[tk], qf[6], s[tk]);
#pragma unroll
    for (int tk = 0; tk < 2; ++tk) s[tk] = mfma32x32x16<T>(kf7[tk], qf[7], s[tk]);
    if constexpr (kLast) stage_out(I3{}, inv);
    stage_end(0, kLast ? 8 : 0);
    pin_products();
    __builtin_amdgcn_s_setprio(0);
    TSTAMP();
    pp_barrier();
    c_slot = n_slot;
    return more;
  };

  // the softmax interval of tile j > 0 of `cur`, up to the barrier; returns nothing, leaves pf, l, vf0, vf1
  // MASKED: the tile the diagonal may cross (the last one; paged: also the one before it when the prefix does not end
  // on a tile boundary, which has a call of its own so that the middle tiles carry no test for it)
  auto later_tile = [&](auto LAST, auto MASKED, auto INSIDE, int j, uint4 (&vf0)[kTD], uint4 (&vf1)[kTD]) {
    TSTAMP();
    if constexpr (decltype(INSIDE)::value) copy_step_inside();
    else copy_step();
    if constexpr (PAGED || HPI != 4) {
      if constexpr (decltype(LAST)::value) mask_tile(j);
      else if constexpr (decltype(MASKED)::value) {
        if (HPI != 4 || (cur.cached & 63) != 0) mask_tile(j);
      }
    } else if constexpr (decltype(LAST)::value) {
      mask_diagonal();
    }
    // The scores are relative to the running maximum, which is not looked at again unless it is badly out of
    // date: the weights are computed first, and only when a lane's share of the tile's row sum passes 2^12 (a
    // weight above 2^7 at least; 16-bit weights and fp32 sums are far from their limits there) is the tile redone
    // the long way: true maximum, accumulators and row sum scaled down, weights again from the kept scores.
    float sum = weights(std::false_type{}, 0.f);
    if (__any(!(sum <= 4096.f))) {
      const float mx = tile_max();
      const float d = mx > 8.f ? mx : 0.f;       // per row (both lanes of a row see the same maximum)
      if (d != 0.f) {
        const float alpha = fast_exp2(-d);
        l *= alpha;
#pragma unroll
        for (int td = 0; td < kTD; ++td)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[td][r] *= alpha;
      }
      set_neg_m(neg_m[0] - d);
      sum = weights(std::true_type{}, d);
    }
    l += sum;
    pin_weights();
    TSTAMP();
    v_frags(c_slot, std::integral_constant<int, 0>{}, vf0);
    v_frags(c_slot, std::integral_constant<int, 1>{}, vf1);
    vm_wait<4>();
    pp_barrier();
    TSTAMP();
  };

  while (true) {
    // ======== first tile of an item ========
    const bool single = cur.nt == 0;
    int trail = 0;                               // vector memory instructions behind this interval's copy step
    TSTAMP();
    copy_step();
    // tiles at the item's end that the diagonal may cross (items of four heads without a prefix: the last one, by
    // mask_diagonal)
    const int masked_tail = kTPB + (PAGED && (cur.cached & 63) != 0 ? 1 : 0);
    if constexpr (PAGED || HPI != 4) {
      if (cur.nt < masked_tail) mask_tile(0);
    } else if (single) {
      mask_diagonal();
    }
    const float mx_first = tile_max();           // neg_m is zero here: the tile's maximum itself
    // the item before this one leaves (its output was staged in the slot during the interval before) ...
    if (have_prev) {
      write_out(p_seq_start, p_seq_len, p_rb, p_h0);
      trail += 8;
    }
    // ... and the next one's Q rows set out
    if (nxt.valid) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot's last readers are done
      copy_q(nxt);
      trail += 8;
    }
    l = weights(std::true_type{}, mx_first);
    set_neg_m(-mx_first);
    uint4 vf0[kTD], vf1[kTD];
    pin_weights();
    TSTAMP();
    v_frags(c_slot, std::integral_constant<int, 0>{}, vf0);   // the tile's first V^T fragments: on their way across the barrier
    v_frags(c_slot, std::integral_constant<int, 1>{}, vf1);
    wait_copies(4 + trail);
    pp_barrier();
    TSTAMP();
    bool more = matrix_interval(std::true_type{}, std::false_type{}, single, vf0, vf1);
    if (!single) {
      // ======== the item's other tiles ========
      if constexpr (HPI == 4) {
        const int plain_end = PAGED ? cur.nt - 1 : cur.nt;
        int j = 1;
        for (; j < cur.nt - 2; ++j) {              // the copy cursor stays inside this item
          later_tile(std::false_type{}, std::false_type{}, std::true_type{}, j, vf0, vf1);
          matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
        }
        for (; j < plain_end; ++j) {
          later_tile(std::false_type{}, std::false_type{}, std::false_type{}, j, vf0, vf1);
          matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
        }
        if constexpr (PAGED) {
          if (cur.nt >= 2) {
            later_tile(std::false_type{}, std::true_type{}, std::false_type{}, cur.nt - 1, vf0, vf1);
            matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
          }
        }
      } else {
        int j = 1;
        for (; j < cur.nt - 2; ++j) {              // the copy cursor stays inside this item (masked_tail >= 2)
          later_tile(std::false_type{}, std::false_type{}, std::true_type{}, j, vf0, vf1);
          matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
        }
        for (; j <= cur.nt - masked_tail; ++j) {
          later_tile(std::false_type{}, std::false_type{}, std::false_type{}, j, vf0, vf1);
          matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
        }
        for (; j < cur.nt; ++j) {                  // one or two tiles before the last that the diagonal crosses
          later_tile(std::false_type{}, std::true_type{}, std::false_type{}, j, vf0, vf1);
          matrix_interval(std::false_type{}, std::false_type{}, false, vf0, vf1);
        }
      }
      later_tile(std::true_type{}, std::true_type{}, std::false_type{}, cur.nt, vf0, vf1);
      more = matrix_interval(std::false_type{}, std::true_type{}, false, vf0, vf1);
    }
    TCOUNT(1, cur.nt + 1);
    p_seq_start = cur.seq_start; p_seq_len = cur.seq_len; p_rb = cur.rb; p_h0 = cur.h0;
    have_prev = true;
    if (!more) break;
    cur = nxt;
    nxt = item_at(ci++);
  }
  if (GRP == 0) pp_barrier();                   // group 1's last interval
  vm_wait<0>();
  write_out(p_seq_start, p_seq_len, p_rb, p_h0);
#if MVLLM_PP_TIMELINE
  if (a.timeline != nullptr && a.timeline_block < 0 && wave == 4 && lane == 0) {
    unsigned long long* e = a.timeline + 4 * (size_t)blockIdx.x;
    e[0] = t_begin;
    e[1] = __builtin_amdgcn_s_memtime();
    e[2] = (unsigned long long)t_items;
    e[3] = (unsigned long long)t_tiles;
  }
#endif
}

template <typename T, int D, bool PAGED, int HPI>
__global__ __launch_bounds__(64 * kPpWaves, 1) void prefill_pp_kernel(const PrefillPpArgs a) {
  __shared__ __attribute__((aligned(1024))) PpLds<D> lds;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (wave < 4) pp_run<T, D, 0, PAGED, HPI>(a, lds, wave);
  else pp_run<T, D, 1, PAGED, HPI>(a, lds, wave);
}

template <typename T>
static void launch_prefill_pp_as(const PrefillPpArgs& a, bool paged, int hpi, dim3 g, dim3 b, hipStream_t stream) {
  if (hpi == 4) {
    if (paged) prefill_pp_kernel<T, 128, true, 4><<<g, b, 0, stream>>>(a);
    else prefill_pp_kernel<T, 128, false, 4><<<g, b, 0, stream>>>(a);
  } else {
    if (paged) prefill_pp_kernel<T, 128, true, 2><<<g, b, 0, stream>>>(a);
    else prefill_pp_kernel<T, 128, false, 2><<<g, b, 0, stream>>>(a);
  }
}

bool prefill_pp_takes(int num_seqs, int num_heads, int num_kv_heads, int head_dim, int dtype, int block_size) {
  if (dtype == MVLLM_F32 || head_dim != 128 || num_seqs > 64 || num_seqs <= 0) return false;
  if (block_size != 0 && (block_size < 16 || block_size % 16 != 0)) return false;      // paged: a wave's 16 rows lie in one block
  if ((int64_t)block_size * num_kv_heads * head_dim * 2 >= ((int64_t)1 << 31)) return false;   // a block's bytes in 32 bits
  const int group = num_heads / num_kv_heads;
  return group % 2 == 0 && (int64_t)num_heads * head_dim * 2 * 64 < ((int64_t)1 << 31);
}

int launch_prefill_pp(const PrefillPpArgs& args, int dtype, hipStream_t stream) {
  PrefillPpArgs a = args;
  const int group = a.num_heads / a.num_kv_heads;
  const int hpi = group % 4 == 0 ? 4 : 2;             // query heads per item
  a.slices = a.num_kv_heads * (group / hpi);
  int n_teams = 8;
  while (a.slices % n_teams != 0) n_teams >>= 1;      // gcd(8, slices)
  a.n_teams = n_teams;
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  const int grid = cus / 8 * 8 > 0 ? cus / 8 * 8 : 8;
  a.team_size = grid / n_teams;
  auto magic = [](int d) { return d <= 1 ? 0u : (unsigned)(((uint64_t)1 << 32) / (uint64_t)d + 1u); };
  a.spt_magic = magic(a.slices / n_teams);
  a.chunks_magic = magic(group / hpi);
  const bool paged = a.block_tables != nullptr;
  a.block_magic = magic(a.block_size);
  a.block_bytes = a.block_size * a.num_kv_heads * 128 * 2;
  a.num_blocks32 = a.num_blocks > 0x7fffffff ? 0x7fffffff : (int)a.num_blocks;
  // levels: one past the last key tile of the longest possible sequence (paged: as wide as its block-table row).  An
  // item of 128 rows counts its tiles from its block's last row, which may lie up to 127 positions past the
  // sequence's last key: three tiles of margin.
  const int64_t most_keys = paged ? (int64_t)a.max_num_blocks * a.block_size + a.total_tokens : a.total_tokens;
  a.level_bits = 1;
  while (((int64_t)1 << a.level_bits) <= most_keys / 64 + 4) ++a.level_bits;
  const dim3 g(grid), b(64 * kPpWaves);
  if (dtype == MVLLM_BF16) launch_prefill_pp_as<bf16_t>(a, paged, hpi, g, b, stream);
  else launch_prefill_pp_as<f16_t>(a, paged, hpi, g, b, stream);
  return launch_status();
}

}  // namespace mvllm

#if MVLLM_PP_TIMELINE
// Probe library only: the two-group prefill with the clock stamps of workgroup `block` written to `log`
// ([8 waves][entries_per_wave] 64-bit shader clocks; entries past a wave's last stamp stay as the caller filled them).
// block < 0: `log` receives {begin, end, items, tiles} of every workgroup instead (4 entries each, grid x 4 in all;
// the grid is the CU count rounded down to a multiple of 8).
extern "C" int mvllm_probe_prefill_timeline(void* out, const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                                            int num_seqs, int64_t total_tokens, int num_heads, int num_kv_heads, int head_dim,
                                            float scale, int dtype, unsigned long long* log, int entries_per_wave, int block,
                                            void* stream) {
  using namespace mvllm;
  if (!out || !q || !k || !v || !cu_seqlens || !log || entries_per_wave <= 0) return MVLLM_ERR_NULL_POINTER;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || !(scale > 0.f) ||
      !prefill_pp_takes(num_seqs, num_heads, num_kv_heads, head_dim, dtype, 0))
    return MVLLM_ERR_UNSUPPORTED;
  PrefillPpArgs p;
  p.out = out; p.q = q; p.k = k; p.v = v; p.cu_seqlens = cu_seqlens; p.total_tokens = total_tokens;
  p.num_seqs = num_seqs; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.scale_log2 = scale * kLog2e;
  p.slices = 0; p.n_teams = 0; p.team_size = 0; p.level_bits = 0; p.spt_magic = 0; p.chunks_magic = 0;
  p.cu_seqlens_k = nullptr; p.block_tables = nullptr; p.max_num_blocks = 0; p.block_size = 0; p.num_blocks = 0; p.block_magic = 0; p.block_bytes = 0; p.num_blocks32 = 0;
  p.timeline = log; p.timeline_entries = entries_per_wave; p.timeline_block = block;
  return launch_prefill_pp(p, dtype, (hipStream_t)stream);
}
#endif
