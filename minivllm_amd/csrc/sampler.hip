// mvllm_sample_tokens: the reference's SamplerLayer.forward (src/myvllm/layers/sampler.py:14-19) in one launch
// and without materialising a (batch, vocab) fp32 probability tensor:
//   logits /= temperature;  probs = softmax(logits);  token = argmax(probs / max(Exp(1) noise, 1e-10))
// softmax is a positive per-row rescaling of exp(logit / T), so the argmax is taken directly over
//   logit / T - log(max(noise, 1e-10))
// (the exponential race / Gumbel-max form of one draw from the tempered distribution).
// The noise is either read from a caller tensor (what the reference's exponential_ call would have produced:
// used by the parity tests) or generated in the kernel with Philox4x32-10, keyed by (seed) and counted by
// (element group, row, call offset), so a (seed, offset) pair always yields the same tokens.
#include <atomic>
#include "common.h"

namespace mvllm {

__device__ __forceinline__ uint4 philox4x32_10(uint4 c, uint2 k) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c.x, p1 = (uint64_t)0xCD9E8D57u * c.z;   // one 32x32->64 multiply each
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    c = make_uint4(hi1 ^ c.y ^ k.x, lo1, hi0 ^ c.w ^ k.y, lo0);
    k.x += 0x9E3779B9u;
    k.y += 0xBB67AE85u;
  }
  return c;
}

// 32 random bits -> uniform in (0, 1): the 24 high bits plus one half, times 2^-24
__device__ __forceinline__ float uniform_open(uint32_t x) { return ((float)(x >> 8) + 0.5f) * 5.9604644775390625e-08f; }

// four consecutive logits as fp32 (one vector load when `vec`), -inf past the end of the row
template <typename T16> __device__ __forceinline__ void load4(const T16* p, bool vec, int n, float (&x)[4]) {
  if (vec) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    x[0] = lo_to_float<T16>(w.x); x[1] = hi_to_float<T16>(w.x);
    x[2] = lo_to_float<T16>(w.y); x[3] = hi_to_float<T16>(w.y);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = e < n ? to_float(p[e]) : -INFINITY;
  }
}
template <> __device__ __forceinline__ void load4<float>(const float* p, bool vec, int n, float (&x)[4]) {
  if (vec) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = e < n ? p[e] : -INFINITY;
  }
}

constexpr int kSampleThreads = 1024;

// better = larger score, ties to the smaller index (first occurrence)
__device__ __forceinline__ void keep_best(float& s, int& i, float s2, int i2) {
  if (s2 > s || (s2 == s && i2 < i)) {
    s = s2;
    i = i2;
  }
}

// One workgroup scans one slice of one row: slices > 1 spreads a row over several workgroups (a small batch
// would otherwise occupy only `batch` CUs with a kernel that is bound by Philox's integer multiplies); each then
// leaves its (score, index) in `partial` and sample_combine_kernel picks the winner.
template <typename T>
__global__ __launch_bounds__(kSampleThreads) void sample_tokens_kernel(
    int64_t* __restrict__ out, float2* __restrict__ partial, const T* __restrict__ logits, int64_t row_stride,
    const float* __restrict__ temperatures, const float* __restrict__ noise, uint32_t seed_lo, uint32_t seed_hi,
    uint32_t off_lo, uint32_t off_hi, const uint64_t* __restrict__ offset_dev, int vocab, int slices) {
  if (offset_dev) {      // the call offset lives on the device (a captured graph cannot change a launch argument)
    const uint64_t off = *offset_dev + (((uint64_t)off_hi << 32) | off_lo);
    off_lo = (uint32_t)off;
    off_hi = (uint32_t)(off >> 32);
  }
  __shared__ float best_s[kSampleThreads / 64];
  __shared__ int best_i[kSampleThreads / 64];
  const int b = blockIdx.x;
  const T* row = logits + (int64_t)b * row_stride;
  const float inv_t = 1.0f / temperatures[b];
  // whole groups of four can be loaded as one vector when the row starts on a vector boundary
  const bool row_vec = ((reinterpret_cast<uintptr_t>(row) & (4 * sizeof(T) - 1)) == 0);
  float s = -INFINITY;
  int idx = 0x7fffffff;
  const int groups = (vocab + 3) >> 2;
  const int per_slice = (groups + slices - 1) / slices;
  const int g_end = min(groups, (int)(blockIdx.y + 1) * per_slice);
  for (int gi = blockIdx.y * per_slice + threadIdx.x; gi < g_end; gi += kSampleThreads) {
    const int i0 = 4 * gi;
    const int n = min(4, vocab - i0);
    float x[4], e[4];
    load4<T>(row + i0, row_vec && n == 4, n, x);
    if (noise) {
#pragma unroll
      for (int k = 0; k < 4; ++k) e[k] = k < n ? noise[(int64_t)b * vocab + i0 + k] : 1.0f;
    } else {
      const uint4 r = philox4x32_10(make_uint4((uint32_t)gi, (uint32_t)b, off_lo, off_hi), make_uint2(seed_lo, seed_hi));
      e[0] = -__logf(uniform_open(r.x));
      e[1] = -__logf(uniform_open(r.y));
      e[2] = -__logf(uniform_open(r.z));
      e[3] = -__logf(uniform_open(r.w));
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float score = x[k] * inv_t - __logf(fmaxf(e[k], 1e-10f));
      if (k < n) keep_best(s, idx, score, i0 + k);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float s2 = __shfl_xor(s, o, 64);
    const int i2 = __shfl_xor(idx, o, 64);
    keep_best(s, idx, s2, i2);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    best_s[wave] = s;
    best_i[wave] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kSampleThreads / 64; ++w) keep_best(s, idx, best_s[w], best_i[w]);
    if (slices == 1) out[b] = idx == 0x7fffffff ? 0 : idx;        // a row of NaNs: token 0
    else partial[(int64_t)b * slices + blockIdx.y] = make_float2(s, __int_as_float(idx));
  }
}

__global__ __launch_bounds__(64) void sample_combine_kernel(int64_t* __restrict__ out, const float2* __restrict__ partial,
                                                            int slices) {
  const int b = blockIdx.x;
  float s = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < slices; i += 64) {
    const float2 p = partial[(int64_t)b * slices + i];
    keep_best(s, idx, p.x, __float_as_int(p.y));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float s2 = __shfl_xor(s, o, 64);
    const int i2 = __shfl_xor(idx, o, 64);
    keep_best(s, idx, s2, i2);
  }
  if (threadIdx.x == 0) out[b] = idx == 0x7fffffff ? 0 : idx;
}

// ---------------------------------------------------------------------------
// LM head + sampler in one pass over the weights: ParallelLMHead.forward (src/myvllm/layers/embedding_head.py:56-77:
// gather the rows to sample from, hidden W^T) and SamplerLayer.forward (layers/sampler.py:14-19) without the
// (batch, vocab) logits ever reaching memory.  The product is a weight stream (151 936 x 1024 bf16 = 311 MB for
// at most 64 rows): a wave owns tiles of 16 vocabulary rows, keeps one to two half tiles (16 rows x K / 2) in flight, and takes
// the hidden rows from LDS, where the workgroup put them once; the logit of (row m, token n) is rounded to the
// element type, as the materialised logits are, scored as in sample_tokens_kernel with the same Philox counter
// (token group n / 4, row, call offset), and only the best (score, token) of every row survives: per lane across
// the wave's tiles, then across the wave, then sample_combine_kernel across the waves of the grid.
// ---------------------------------------------------------------------------
struct LmHeadArgs {
  int64_t* out;
  float2* partial;            // [batch, workgroups]: every workgroup's best (score, token) per row
  const void* hidden;
  int64_t hidden_stride;      // elements between rows of hidden
  const int64_t* row_index;   // [batch] rows of hidden to sample from, or null: rows 0 .. batch-1
  const void* weight;         // [vocab, K]
  const float* temperatures;
  const uint64_t* offset_dev;
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  int batch, vocab, K, slices;   // slices: waves in the grid (the stride of a wave's tiles)
};

constexpr int kLmPad = 8;       // elements of padding per LDS row: rows 16 bytes off the bank stride

template <typename T, int MT, int KS, int kLmWaves>      // MT row tiles of 16, KS 32-wide k steps (K = 32 KS), waves per workgroup
__global__ __launch_bounds__(64 * kLmWaves) void lm_head_sample_kernel(const LmHeadArgs a) {
  extern __shared__ __align__(16) unsigned char lm_smem[];
  T* xs = reinterpret_cast<T*>(lm_smem);                  // [16 MT][K + kLmPad]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, cls = lane >> 4;
  const int K = 32 * KS, ldk = K + kLmPad;
  uint32_t off_lo = a.off_lo, off_hi = a.off_hi;
  if (a.offset_dev) {
    const uint64_t off = *a.offset_dev + (((uint64_t)off_hi << 32) | off_lo);
    off_lo = (uint32_t)off;
    off_hi = (uint32_t)(off >> 32);
  }
  // A wave's tiles are 16 vocabulary rows each; the two halves of a tile's K are loaded as separate bursts, and
  // the burst of the next tile's half is asked for as soon as this tile's half has been consumed, so a wave always
  // has 16 to 32 rows x K / 2 in flight.  The first tile is asked for before the hidden rows are staged.
  constexpr int KH = KS / 2;
  const int tiles = a.vocab / 16;
  const int wave_id = blockIdx.x * kLmWaves + wave;
  const T* wbase = reinterpret_cast<const T*>(a.weight) + (int64_t)col * K + 8 * cls;
  uint4 wa[KH], wb[KH];
  auto ask = [&](uint4 (&w)[KH], int t, int half) __attribute__((always_inline)) {
    const T* wp = wbase + (int64_t)t * 16 * K + half * (K / 2);
#pragma unroll
    for (int ks = 0; ks < KH; ++ks) w[ks] = load16_stream(wp + 32 * ks);
  };
  int t = wave_id;
  if (t < tiles) {
    ask(wa, t, 0);
    ask(wb, t, 1);
  }
  // the hidden rows, once per workgroup (rows past the batch repeat the last one and are never scored)
  for (int i = threadIdx.x; i < 16 * MT * (K / 8); i += 64 * kLmWaves) {
    const int m = i / (K / 8), c = i - m * (K / 8);
    const int mm = min(m, a.batch - 1);
    const int64_t r = a.row_index ? a.row_index[mm] : mm;
    *reinterpret_cast<uint4*>(xs + m * ldk + 8 * c) =
        *reinterpret_cast<const uint4*>(reinterpret_cast<const T*>(a.hidden) + r * a.hidden_stride + 8 * c);
  }
  float inv_t[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) inv_t[mt] = 1.0f / a.temperatures[min(16 * mt + col, a.batch - 1)];
  __syncthreads();

  float best_s[MT];
  int best_i[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    best_s[mt] = -INFINITY;
    best_i[mt] = 0x7fffffff;
  }
  v4f acc[MT];
  auto consume = [&](const uint4 (&w)[KH], int half) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < KH; ++ks) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const uint4 xf = *reinterpret_cast<const uint4*>(xs + (16 * mt + col) * ldk + half * (K / 2) + 32 * ks + 8 * cls);
        acc[mt] = mfma16x16x32<T>(w[ks], xf, acc[mt]);
      }
      // keep the LDS reads of later steps behind this one: hoisted to the top they cost MT x KS x 4 registers
      if (MT * (ks + 1) % 8 == 0) __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (; t < tiles; t += a.slices) {
    const int tn = t + a.slices;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = (v4f){0.f, 0.f, 0.f, 0.f};
    consume(wa, 0);
    if (tn < tiles) ask(wa, tn, 0);
    consume(wb, 1);
    if (tn < tiles) ask(wb, tn, 1);
    // lane l holds the logits of row m = 16 mt + l % 16 for tokens 16 t + 4 (l / 16) + r: one Philox group each
    const int gi = 4 * t + cls;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = 16 * mt + col;
      if (m < a.batch) {
        const uint4 rnd = philox4x32_10(make_uint4((uint32_t)gi, (uint32_t)m, off_lo, off_hi), make_uint2(a.seed_lo, a.seed_hi));
        const float e[4] = {-__logf(uniform_open(rnd.x)), -__logf(uniform_open(rnd.y)), -__logf(uniform_open(rnd.z)),
                            -__logf(uniform_open(rnd.w))};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float logit = to_float(from_float<T>(acc[mt][r]));          // the logits tensor is in the element type
          const float score = logit * inv_t[mt] - __logf(fmaxf(e[r], 1e-10f));
          keep_best(best_s[mt], best_i[mt], score, 4 * gi + r);
        }
      }
    }
  }
  // the four lanes of a row, then the four waves of the workgroup (through LDS, where the hidden rows are no longer
  // needed), then this workgroup's entry of the row's partials
  __syncthreads();
  float2* wg_best = reinterpret_cast<float2*>(lm_smem);        // [kLmWaves][16 MT]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int o = 16; o <= 32; o <<= 1) {
      const float s2 = __shfl_xor(best_s[mt], o, 64);
      const int i2 = __shfl_xor(best_i[mt], o, 64);
      keep_best(best_s[mt], best_i[mt], s2, i2);
    }
    if (cls == 0) wg_best[wave * 16 * MT + 16 * mt + col] = make_float2(best_s[mt], __int_as_float(best_i[mt]));
  }
  __syncthreads();
  for (int m = threadIdx.x; m < a.batch; m += 64 * kLmWaves) {
    float sb = -INFINITY;
    int ib = 0x7fffffff;
    for (int w = 0; w < kLmWaves; ++w) {
      const float2 p = wg_best[w * 16 * MT + m];
      keep_best(sb, ib, p.x, __float_as_int(p.y));
    }
    a.partial[(int64_t)m * gridDim.x + blockIdx.x] = make_float2(sb, __int_as_float(ib));
  }
}

// workgroups of the LM-head pass: two of four waves per CU while the hidden rows leave room for two in LDS, else one
// of eight waves
static int lm_head_groups(int batch, int K) {
  const size_t lds = (size_t)((batch + 15) / 16 * 16) * (size_t)(K + kLmPad) * 2;
  return lds <= 72 * 1024 ? 512 : 256;
}
static int lm_head_waves(int batch, int K) { return lm_head_groups(batch, K) == 512 ? 4 : 8; }

template <typename T, int MT, int W>
static int launch_lm_head(const LmHeadArgs& a, int groups, size_t lds, hipStream_t s) {
  const dim3 grid((unsigned)groups), block(64 * W);
#define MVLLM_LM(KS_)                                                                                         \
  do {                                                                                                        \
    static std::atomic<int> allowed{0};          /* dynamic LDS this instantiation has been allowed so far */ \
    if (lds > 48 * 1024 && (int)lds > allowed.load(std::memory_order_relaxed)) {                              \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&lm_head_sample_kernel<T, MT, KS_, W>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
      if (e != hipSuccess) return (int)e;                                                                     \
      allowed.store((int)lds, std::memory_order_relaxed);                                                     \
    }                                                                                                         \
    lm_head_sample_kernel<T, MT, KS_, W><<<grid, block, lds, s>>>(a);                                         \
  } while (0)
  switch (a.K / 32) {
    case 8: MVLLM_LM(8); break;
    case 16: MVLLM_LM(16); break;
    case 32: MVLLM_LM(32); break;
    default: return MVLLM_ERR_UNSUPPORTED;
  }
#undef MVLLM_LM
  return launch_status();
}

}  // namespace mvllm

using namespace mvllm;

extern "C" size_t mvllm_sample_tokens_workspace_bytes(int batch, int vocab) {
  if (batch <= 0 || vocab <= 0) return 0;
  // enough slices for about two workgroups per CU, each with at least 4096 logits
  int slices = (512 + batch - 1) / batch;
  const int max_slices = (vocab + 4095) / 4096;
  if (slices > max_slices) slices = max_slices;
  return slices <= 1 ? 0 : (size_t)batch * (size_t)slices * sizeof(float2);
}

static int sample_entry(int64_t* out_ids, const void* logits, int64_t row_stride, const float* temperatures,
                        const float* noise, uint64_t seed, uint64_t offset, const uint64_t* offset_dev, int batch,
                        int vocab, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  const int esize = dtype_size(dtype);
  if (esize == 0) return MVLLM_ERR_BAD_DTYPE;
  if (batch < 0 || vocab <= 0 || row_stride < vocab) return MVLLM_ERR_BAD_SHAPE;
  if (batch == 0) return MVLLM_OK;
  if (!out_ids || !logits || !temperatures) return MVLLM_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(logits) & (uintptr_t)(esize - 1)) != 0) return MVLLM_ERR_MISALIGNED;
  // a row is split over as many workgroups as the workspace has room for (none: one workgroup per row)
  const size_t want = mvllm_sample_tokens_workspace_bytes(batch, vocab);
  int slices = 1;
  if (workspace && want > 0 && workspace_bytes >= want) {
    if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return MVLLM_ERR_WORKSPACE;
    slices = (int)(want / ((size_t)batch * sizeof(float2)));
  }
  hipStream_t s = (hipStream_t)stream;
  const uint32_t sl = (uint32_t)seed, sh = (uint32_t)(seed >> 32), ol = (uint32_t)offset, oh = (uint32_t)(offset >> 32);
  const dim3 grid((unsigned)batch, (unsigned)slices), block(kSampleThreads);
  float2* part = reinterpret_cast<float2*>(workspace);
  switch (dtype) {
    case MVLLM_F32:
      sample_tokens_kernel<float><<<grid, block, 0, s>>>(out_ids, part, (const float*)logits, row_stride, temperatures,
                                                        noise, sl, sh, ol, oh, offset_dev, vocab, slices);
      break;
    case MVLLM_BF16:
      sample_tokens_kernel<bf16_t><<<grid, block, 0, s>>>(out_ids, part, (const bf16_t*)logits, row_stride, temperatures,
                                                         noise, sl, sh, ol, oh, offset_dev, vocab, slices);
      break;
    default:
      sample_tokens_kernel<f16_t><<<grid, block, 0, s>>>(out_ids, part, (const f16_t*)logits, row_stride, temperatures,
                                                        noise, sl, sh, ol, oh, offset_dev, vocab, slices);
      break;
  }
  if (slices > 1) sample_combine_kernel<<<dim3((unsigned)batch), dim3(64), 0, s>>>(out_ids, part, slices);
  return launch_status();
}

extern "C" int mvllm_sample_tokens(int64_t* out_ids, const void* logits, int64_t row_stride,
                                   const float* temperatures, const float* noise, uint64_t seed, uint64_t offset,
                                   int batch, int vocab, int dtype, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  return sample_entry(out_ids, logits, row_stride, temperatures, noise, seed, offset, nullptr, batch, vocab, dtype,
                      workspace, workspace_bytes, stream);
}

extern "C" int mvllm_sample_tokens_dev_offset(int64_t* out_ids, const void* logits, int64_t row_stride,
                                              const float* temperatures, uint64_t seed, const uint64_t* offset_dev,
                                              int batch, int vocab, int dtype, void* workspace,
                                              size_t workspace_bytes, void* stream) {
  if (!offset_dev) return MVLLM_ERR_NULL_POINTER;
  return sample_entry(out_ids, logits, row_stride, temperatures, nullptr, seed, 0, offset_dev, batch, vocab, dtype,
                      workspace, workspace_bytes, stream);
}

// ---------------------------------------------------------------------------
// The step metadata of a decode batch that continues the step before it (the same sequences, each one token longer),
// moved forward on the device: next input = the id just sampled, context length, position and slot + 1.  One launch
// in place of the host rebuilding and copying the four tensors (ModelRunner.prepare_decode,
// src/myvllm/engine/model_runner.py:231-256).  Rows whose context length is not positive are padding of a captured
// batch size and stay as they are; `step` (optional) is the sampler's call counter, incremented once per launch, so
// that a captured decode step ends with everything the next replay needs; `host_ids` (optional, with `step`): two
// rows of `host_stride` int64 in pinned host memory; row r = (counter before the increment) & 1 receives the sampled
// ids in its first `n` entries and then, behind a system-scope fence, the new counter value in its last entry.  The
// host reads a step's ids as soon as it sees that value: no copy operation and no event between two replays (an
// event record between two graph launches costs 12 to 30 us here).
// One workgroup (every thread reads the counter before thread 0 moves it).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void decode_advance_kernel(int64_t* __restrict__ input_ids, int64_t* __restrict__ context_lens,
                                                             int64_t* __restrict__ positions, int64_t* __restrict__ slot_mapping,
                                                             const int64_t* __restrict__ sampled, uint64_t* __restrict__ step,
                                                             int64_t* __restrict__ host_ids, int64_t host_stride, int n) {
  const uint64_t before = step ? *step : 0;
  __syncthreads();
  if (threadIdx.x == 0 && step) *step = before + 1;
  int64_t* host_row = host_ids ? host_ids + (int64_t)(before & 1u) * host_stride : nullptr;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int64_t id = sampled[i];
    if (host_row) host_row[i] = id;
    const int64_t ctx = context_lens[i];
    if (ctx <= 0) continue;
    input_ids[i] = id;
    context_lens[i] = ctx + 1;
    positions[i] = ctx;
    slot_mapping[i] += 1;
  }
  if (host_row) {
    __threadfence_system();                  // every thread's ids are in host memory ...
    __syncthreads();
    if (threadIdx.x == 0) {                  // ... before the value that says so
      __hip_atomic_store(reinterpret_cast<uint64_t*>(host_row + host_stride - 1), before + 1, __ATOMIC_RELEASE,
                         __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

extern "C" int mvllm_decode_advance(int64_t* input_ids, int64_t* context_lens, int64_t* positions,
                                    int64_t* slot_mapping, const int64_t* sampled, uint64_t* step_counter,
                                    int64_t* host_ids, int64_t host_row_stride, int batch, void* stream) {
  if (batch < 0 || (host_ids && host_row_stride < (int64_t)batch + 1)) return MVLLM_ERR_BAD_SHAPE;
  if (host_ids && !step_counter) return MVLLM_ERR_NULL_POINTER;
  if (batch == 0 && !step_counter) return MVLLM_OK;
  if (batch > 0 && (!input_ids || !context_lens || !positions || !slot_mapping || !sampled)) return MVLLM_ERR_NULL_POINTER;
  decode_advance_kernel<<<dim3(1), dim3(256), 0, (hipStream_t)stream>>>(input_ids, context_lens, positions, slot_mapping,
                                                                        sampled, step_counter, host_ids, host_row_stride, batch);
  return launch_status();
}

extern "C" size_t mvllm_lm_head_sample_workspace_bytes(int batch, int K) {
  if (batch <= 0 || batch > 64 || K <= 0) return 0;
  return (size_t)batch * (size_t)lm_head_groups(batch, K) * sizeof(float2);
}

extern "C" int mvllm_lm_head_sample(int64_t* out_ids, const void* hidden, int64_t hidden_row_stride,
                                    const int64_t* row_index, const void* weight, const float* temperatures,
                                    uint64_t seed, uint64_t offset, const uint64_t* offset_dev, int batch, int vocab,
                                    int K, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != MVLLM_BF16 && dtype != MVLLM_F16) return dtype_size(dtype) == 0 ? MVLLM_ERR_BAD_DTYPE : MVLLM_ERR_UNSUPPORTED;
  if (batch < 0 || vocab <= 0 || K <= 0 || hidden_row_stride < K) return MVLLM_ERR_BAD_SHAPE;
  if (batch == 0) return MVLLM_OK;
  if (!out_ids || !hidden || !weight || !temperatures) return MVLLM_ERR_NULL_POINTER;
  if (batch > 64 || vocab % 16 != 0 || (K != 256 && K != 512 && K != 1024) || hidden_row_stride % 8 != 0)
    return MVLLM_ERR_UNSUPPORTED;
  if (!aligned16(hidden) || !aligned16(weight)) return MVLLM_ERR_MISALIGNED;
  const size_t need = mvllm_lm_head_sample_workspace_bytes(batch, K);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return MVLLM_ERR_WORKSPACE;
  LmHeadArgs a;
  a.out = out_ids; a.partial = reinterpret_cast<float2*>(workspace);
  a.hidden = hidden; a.hidden_stride = hidden_row_stride; a.row_index = row_index; a.weight = weight;
  a.temperatures = temperatures; a.offset_dev = offset_dev;
  a.seed_lo = (uint32_t)seed; a.seed_hi = (uint32_t)(seed >> 32);
  a.off_lo = (uint32_t)offset; a.off_hi = (uint32_t)(offset >> 32);
  a.batch = batch; a.vocab = vocab; a.K = K;
  const int groups = lm_head_groups(batch, K);
  const int waves = lm_head_waves(batch, K);
  a.slices = groups * waves;
  const int mt = (batch + 15) / 16;
  const size_t lds = (size_t)(16 * mt) * (size_t)(K + kLmPad) * 2;
  hipStream_t s = (hipStream_t)stream;
  int st;
#define MVLLM_LM_T(T_)                                                                                          \
  (waves == 4 ? (mt == 1   ? launch_lm_head<T_, 1, 4>(a, groups, lds, s)                                        \
                 : mt == 2 ? launch_lm_head<T_, 2, 4>(a, groups, lds, s)                                        \
                 : mt == 3 ? launch_lm_head<T_, 3, 4>(a, groups, lds, s)                                        \
                           : launch_lm_head<T_, 4, 4>(a, groups, lds, s))                                       \
              : (mt == 1   ? launch_lm_head<T_, 1, 8>(a, groups, lds, s)                                        \
                 : mt == 2 ? launch_lm_head<T_, 2, 8>(a, groups, lds, s)                                        \
                 : mt == 3 ? launch_lm_head<T_, 3, 8>(a, groups, lds, s)                                        \
                           : launch_lm_head<T_, 4, 8>(a, groups, lds, s)))
  st = dtype == MVLLM_BF16 ? MVLLM_LM_T(bf16_t) : MVLLM_LM_T(f16_t);
#undef MVLLM_LM_T
  if (st != 0) return st;
  sample_combine_kernel<<<dim3((unsigned)batch), dim3(64), 0, s>>>(out_ids, a.partial, groups);
  return launch_status();
}
