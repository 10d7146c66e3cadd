/*
 * minivllm_amd.h -- C ABI of libminivllm_amd.so (gfx950 / MI355X).
 *
 * The reference (Wenyueh/MinivLLM) is pure Python + Triton and has no FFI;
 * each entry point below replaces the Triton launch inside one of the
 * reference's Python operators and is what a ctypes binding of that operator
 * calls.  The reference location of the operator is cited per function.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - return value: 0 ok, <0 invalid argument / unsupported shape
 *     (see mvllm_status_string), >0 a hipError_t from the launch;
 *   - the library never allocates, frees or synchronises; outputs and
 *     workspaces are caller-owned; launches have static grids derived from the
 *     host arguments only, so every call is legal under hipGraph capture;
 *   - tensors are dense row-major ("contiguous") in the stated shape.
 */
#ifndef MINIVLLM_AMD_H_
#define MINIVLLM_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of q/k/v/out and of a non-quantised KV cache */
enum mvllm_dtype {
  MVLLM_F32 = 0,
  MVLLM_BF16 = 1,
  MVLLM_F16 = 2,
};

/* negative status codes */
enum mvllm_status {
  MVLLM_OK = 0,
  MVLLM_ERR_NULL_POINTER = -1,
  MVLLM_ERR_BAD_DTYPE = -2,
  MVLLM_ERR_BAD_SHAPE = -3,      /* a size is <= 0 where it must be positive, or not divisible as required */
  MVLLM_ERR_UNSUPPORTED = -4,    /* shape valid but no kernel is built for it */
  MVLLM_ERR_WORKSPACE = -5,      /* workspace missing or smaller than *_workspace_bytes() */
  MVLLM_ERR_MISALIGNED = -6,     /* pointer not aligned to 16 bytes */
};

/* ABI version: major*1000 + minor. */
int mvllm_version(void);

/* Static, human-readable text for a status returned by this library
 * (negative codes only; positive codes are hipError_t). HOST pointer. */
const char* mvllm_status_string(int status);

/*
 * store_kvcache -- src/myvllm/layers/attention.py:67-108 (kernel :7-64).
 * For every token t with slot = slot_mapping[t]:
 *     slot == -1 (or outside [0, num_slots))  -> nothing is written
 *     else k_cache_flat[slot, :, :] = key[t, :, :], same for value,
 * where *_cache_flat is the [num_slots = num_blocks*block_size, Hkv, D] view of
 * the [num_blocks, block_size, Hkv, D] cache.  key/value: [T, Hkv, D], same
 * dtype as the caches (a bit-exact copy).  slot_mapping: int64 [T].
 */
int mvllm_store_kvcache(const void* key, const void* value,
                        void* k_cache, void* v_cache,
                        const int64_t* slot_mapping,
                        int64_t num_tokens, int64_t num_slots,
                        int num_kv_heads, int head_dim,
                        int dtype, void* stream);

/*
 * INT8 variant of store_kvcache (no counterpart in the reference; it serves
 * the same call site, attention.py:510, when the cache is int8).
 * Per (token, kv head): amax = max|x| in fp32, scale = amax / 127 (IEEE fp32
 * divide), code = clamp(rint(x / scale), -127, 127) (round half to even);
 * amax == 0 -> scale 0, codes 0.  Codes go to int8 caches [num_slots, Hkv, D],
 * scales to fp32 [num_slots, Hkv].  `dtype` is the dtype of key/value.
 */
int mvllm_store_kvcache_int8(const void* key, const void* value,
                             int8_t* k_cache, int8_t* v_cache,
                             float* k_scale, float* v_scale,
                             const int64_t* slot_mapping,
                             int64_t num_tokens, int64_t num_slots,
                             int num_kv_heads, int head_dim,
                             int dtype, void* stream);

/*
 * Bytes of fp32 split-K workspace mvllm_paged_decode{,_int8} need for these
 * static sizes (0 if the shape needs none).  Pure host arithmetic.
 */
size_t mvllm_paged_decode_workspace_bytes(int batch, int num_heads, int head_dim,
                                          int max_num_blocks, int block_size);

/*
 * How mvllm_paged_decode{,_int8} split these static sizes (no counterpart in the reference, whose Triton kernel
 * walks a whole context in one program, attention.py:283-415).  Pure host arithmetic:
 *   *part_tokens      tokens of a partition; partition p of a sequence covers tokens [p, p+1) * part_tokens
 *   *num_parts        partitions per sequence (1: no workspace is touched and no merge kernel is launched)
 *   *waves_per_head   1: a workgroup holds up to 4 kv heads, one wave each, and every wave walks its partition;
 *                     >1: small-batch form, a workgroup is that many waves on one kv head that share the
 *                     partition's 16-token tiles and merge in LDS; 0: the generic kernel (head_dim other than
 *                     128 or 64 (bf16 / fp16 caches: also every other multiple of 8 from 32 to 120, and 256),
 *                     a block_size that is neither a multiple of 16 nor, for 16-bit and fp32 caches with head_dim 128 or
 *                     64, one of 1, 2, 4, 8; or fp32 queries over an INT8 cache).  A kv head with more than 16 query
 *                     heads is served in slices of 16, each of which streams its keys and values again.
 * Returns MVLLM_OK or MVLLM_ERR_BAD_SHAPE / MVLLM_ERR_BAD_DTYPE.
 */
int mvllm_paged_decode_plan(int batch, int num_heads, int num_kv_heads, int head_dim,
                            int max_num_blocks, int block_size, int dtype, int int8_cache,
                            int* part_tokens, int* num_parts, int* waves_per_head);

/*
 * paged_attention_decode -- src/myvllm/layers/attention.py:418-473 (kernel :283-415).
 * out[b,h,:] = softmax_t( scale * q[b,h,:] . K[b,t,g(h),:] ) V[b,t,g(h),:],
 * t in [0, context_lens[b]), g(h) = h / (Hq/Hkv); token t of sequence b lives at
 * cache[block_tables[b, t / block_size], t % block_size, g, :].
 * Tokens whose table index is >= max_num_blocks, or whose entry is < 0 or
 * >= num_blocks, contribute nothing; context_len <= 0 gives a row of zeros.
 *   out, q        [batch, Hq, D]  `dtype`
 *   k/v_cache     [num_blocks, block_size, Hkv, D]  `dtype`
 *   block_tables  int32 [batch, max_num_blocks]
 *   context_lens  int64 [batch] if ctx_is_i64 else int32 [batch]
 *   workspace     >= mvllm_paged_decode_workspace_bytes(...) bytes, 16-byte aligned
 */
int mvllm_paged_decode(void* out, const void* q,
                       const void* k_cache, const void* v_cache,
                       const int32_t* block_tables, int max_num_blocks,
                       const void* context_lens, int ctx_is_i64,
                       int batch, int num_heads, int num_kv_heads, int head_dim,
                       int block_size, int64_t num_blocks, float scale, int dtype,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * INT8-cache variant of paged decode (no counterpart in the reference).
 * K/V rows are dequantised in-kernel as code * scale in fp32.
 *   k/v_cache  int8 [num_blocks, block_size, Hkv, D]
 *   k/v_scale  fp32 [num_blocks, block_size, Hkv]
 *   `dtype` is the dtype of q and out.
 */
int mvllm_paged_decode_int8(void* out, const void* q,
                            const int8_t* k_cache, const int8_t* v_cache,
                            const float* k_scale, const float* v_scale,
                            const int32_t* block_tables, int max_num_blocks,
                            const void* context_lens, int ctx_is_i64,
                            int batch, int num_heads, int num_kv_heads, int head_dim,
                            int block_size, int64_t num_blocks, float scale, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * mvllm_paged_decode for callers that cannot allocate device memory (code under hipGraph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * mvllm_paged_decode without the workspace: the split-K partials go to a static device array inside the library
 * (MVLLM_PAGED_DECODE_NOALLOC_MAX_BYTES per GPU, held until the process ends).  Shapes for which
 * mvllm_paged_decode_workspace_bytes() exceeds that size return MVLLM_ERR_WORKSPACE.  The call allocates and frees
 * nothing; the first call on a device looks up the array's address (make it outside graph capture).  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams, two threads) race on it.  Nothing in it
 * has to be cleared between calls: a merge reads only partials that the same call has written.
 */
#define MVLLM_PAGED_DECODE_NOALLOC_MAX_BYTES (32u << 20)
int mvllm_paged_decode_noalloc(void* out, const void* q,
                               const void* k_cache, const void* v_cache,
                               const int32_t* block_tables, int max_num_blocks,
                               const void* context_lens, int ctx_is_i64,
                               int batch, int num_heads, int num_kv_heads, int head_dim,
                               int block_size, int64_t num_blocks, float scale, int dtype,
                               void* stream);

/*
 * flash_attention_prefill -- src/myvllm/layers/attention.py:212-280 (kernel :111-209).
 * Packed ragged batch: sequence s owns rows [cu_seqlens[s], cu_seqlens[s+1]).
 * out[i,h,:] = softmax_{j<=i, same sequence}( scale * q[i,h,:] . k[j,g(h),:] ) v[j,g(h),:].
 *   out, q  [T, Hq, D];  k, v  [T, Hkv, D];  cu_seqlens int32 [num_seqs+1]
 * Needs no maximum sequence length: the grid is sized from total_tokens and
 * num_seqs (the reference synchronises with the host to find it, :263-264).
 */
int mvllm_prefill_varlen(void* out, const void* q, const void* k, const void* v,
                         const int32_t* cu_seqlens, int num_seqs, int64_t total_tokens,
                         int num_heads, int num_kv_heads, int head_dim,
                         float scale, int dtype, void* stream);

/*
 * Which kernel a prefill of these static sizes runs on (no counterpart in the reference, whose Triton kernels take any
 * power-of-two head_dim from a tile-size table, attention.py:249-257).  block_size 0 = the packed entry point,
 * > 0 = the paged ones.  *kernel: 2 an LDS-tiled MFMA kernel (bf16 / fp16 with a head_dim that is a multiple of 8 from
 * 32 to 128, or 256; fp32 with 128 or 64; over an INT8 cache 64 or 128; the packed and the 16-bit paged entry point run its
 * two-group form where head_dim is 128, the query heads per kv head are an even number and the batch has at most 64
 * sequences), 1 the 16-row tile MFMA kernel (a paged cache whose blocks hold 2^31 bytes or more), 0 the generic kernel (any
 * head_dim <= 512; one key per step, a correctness path two orders of magnitude slower), -1 unsupported.
 * Pointers are assumed 16-byte aligned (unaligned ones take the generic kernel).  Pure host arithmetic.
 */
int mvllm_prefill_plan(int num_heads, int num_kv_heads, int head_dim, int block_size, int dtype,
                       int int8_cache, int* kernel);

/*
 * Prefill over a paged cache: the same attention as mvllm_prefill_varlen for sequences whose first tokens are
 * already in the cache (prefix-cache hits).  The reference prepares exactly this metadata in
 * ModelRunner.prepare_prefill (src/myvllm/engine/model_runner.py:192-226: input_ids = tokens[num_cached:],
 * cu_seqlens_q over the new tokens, cu_seqlens_k over all of them, block_tables when they differ) but its
 * Attention.forward never consumes it (attention.py:518-523 passes cu_seqlens_q and the fresh k, v only).
 *   q, out       [total_q_tokens, Hq, D]: rows of the new tokens only, packed by cu_seqlens_q
 *   k/v_cache    [num_blocks, block_size, Hkv, D], already holding every key of every sequence
 *                (prefix from earlier requests, new tokens from the store that precedes this call)
 *   block_tables int32 [num_seqs, max_num_blocks]; cu_seqlens_q/k int32 [num_seqs+1]
 * Query row r of sequence s (r counted over its new tokens) sits at position
 * c_s + r, c_s = len_k(s) - len_q(s), and attends keys 0 .. c_s + r.  The first ceil(len_k/bs) table
 * entries of a sequence are expected to be valid; an entry < 0 or >= num_blocks there is not followed (no
 * out-of-range access): its keys and values read as zeros.  With c_s = 0 for every s the result equals
 * mvllm_prefill_varlen bit for bit (block sizes that are multiples of 16: both calls then run the same kernel).
 */
int mvllm_prefill_paged(void* out, const void* q, const void* k_cache, const void* v_cache,
                        const int32_t* block_tables, int max_num_blocks,
                        const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                        int num_seqs, int64_t total_q_tokens,
                        int num_heads, int num_kv_heads, int head_dim, int block_size,
                        int64_t num_blocks, float scale, int dtype, void* stream);

/*
 * The same prefill over an INT8 cache (codes + fp32 scales per (token, kv head), as mvllm_store_kvcache_int8 writes
 * them; no counterpart in the reference, which has neither an INT8 cache nor a consumer of its prefix-cache
 * metadata).  Every key, the new tokens' included, is read from the cache and dequantised (code * scale, rounded
 * to `dtype`) on the way into the matrix unit, which is what decode will see for the same tokens.
 * bf16 / fp16 queries, head_dim 128 or 64, block_size a multiple of 16; else MVLLM_ERR_UNSUPPORTED.
 */
int mvllm_prefill_paged_int8(void* out, const void* q,
                             const int8_t* k_cache, const int8_t* v_cache,
                             const float* k_scale, const float* v_scale,
                             const int32_t* block_tables, int max_num_blocks,
                             const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                             int num_seqs, int64_t total_q_tokens,
                             int num_heads, int num_kv_heads, int head_dim, int block_size,
                             int64_t num_blocks, float scale, int dtype, void* stream);

/*
 * mvllm_prefill_paged and mvllm_prefill_paged_int8 in two steps, for callers that can lend device memory: every
 * sequence's keys and values are first written into `workspace`, laid out as a 16-bit paged cache of 16-token blocks with
 * a block table of its own, and the two-group prefill kernel (shapes it does not take: the one-group kernel's 16-bit
 * paged form) runs over that.  No counterpart in the reference.  Two uses:
 *   - an INT8 cache: a value is dequantised once (the same code * scale rounded to `dtype`), where the one-step form
 *     converts a K/V tile again for every query tile that walks it;
 *   - any block_size >= 1: the one-step forms need a multiple of 16 for their MFMA kernels.
 *   max_kv_len     an upper bound of every sequence's len_k, known to the host (the reference's Context.max_seqlen_k,
 *                  utils/context.py:11); keys of a sequence past it read as zeros
 *   workspace      256-byte aligned, at least mvllm_prefill_paged_staged_workspace_bytes(...) bytes; contents need not
 *                  be kept between calls; calls that share a workspace must not overlap
 * mvllm_prefill_paged_staged_workspace_bytes returns 0 for shapes this form is not built for (it takes bf16 / fp16 with
 * head_dim 128 or 64, 16-bit caches also 32, 48, 80, 96, 112 and 256); the entry points then return
 * MVLLM_ERR_UNSUPPORTED and the one-step form is the one to call.
 * Other arguments and the result's meaning as for the one-step forms; MVLLM_ERR_WORKSPACE for a workspace that is null,
 * too small or misaligned.
 */
size_t mvllm_prefill_paged_staged_workspace_bytes(int num_seqs, int max_kv_len, int num_heads, int num_kv_heads,
                                                  int head_dim, int dtype, int int8_cache);
int mvllm_prefill_paged_staged(void* out, const void* q, const void* k_cache, const void* v_cache,
                               const int32_t* block_tables, int max_num_blocks,
                               const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               int num_seqs, int64_t total_q_tokens, int max_kv_len,
                               int num_heads, int num_kv_heads, int head_dim, int block_size,
                               int64_t num_blocks, float scale, int dtype,
                               void* workspace, size_t workspace_bytes, void* stream);
int mvllm_prefill_paged_int8_staged(void* out, const void* q,
                                    const int8_t* k_cache, const int8_t* v_cache,
                                    const float* k_scale, const float* v_scale,
                                    const int32_t* block_tables, int max_num_blocks,
                                    const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                    int num_seqs, int64_t total_q_tokens, int max_kv_len,
                                    int num_heads, int num_kv_heads, int head_dim, int block_size,
                                    int64_t num_blocks, float scale, int dtype,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * mvllm_prefill_paged with every sequence's keys cut into `splits` ranges that are walked side by side and merged: for
 * batches of few new tokens behind long cached prefixes (a follow-up turn, the last chunk of a chunked prefill), whose
 * few query tiles would each walk a whole prefix while most of the chip idles.  No counterpart in the reference (its
 * prefill never reads the paged cache, src/myvllm/layers/attention.py:111-209, and the prefix-hit metadata that
 * model_runner.py:192-226 builds goes unused, attention.py:518-523).
 * 16-bit caches at the head dims of the LDS-tiled kernel (64, 128; 32, 48, 80, 96, 112, 256), INT8 caches
 * (mvllm_prefill_paged_int8_split: codes + scales as for mvllm_prefill_paged_int8) at head_dim 64 and 128; block_size a
 * multiple of 16, num_seqs * splits <= 64.
 *   _split_plan: the number of ranges the library would use for a batch of these sizes; 0 = run mvllm_prefill_paged.
 *   _split_workspace_bytes: 256-byte aligned device memory the call needs for `splits` ranges (range tables, partial
 *     results [splits, total_q_tokens, Hq, D] and their softmax denominators); 0 = shape not taken.
 * max_kv_len: the host's upper bound of every sequence's key count, as in the staged forms.  Results differ from the
 * one-step form's by the rounding of the partial results to the element type (within the same tolerance).
 */
int mvllm_prefill_paged_split_plan(int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                   int num_kv_heads, int head_dim, int block_size, int dtype, int int8_cache);
size_t mvllm_prefill_paged_split_workspace_bytes(int num_seqs, int64_t total_q_tokens, int max_kv_len, int num_heads,
                                                 int num_kv_heads, int head_dim, int block_size, int dtype, int splits);
int mvllm_prefill_paged_split(void* out, const void* q, const void* k_cache, const void* v_cache,
                              const int32_t* block_tables, int max_num_blocks,
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                              int num_seqs, int64_t total_q_tokens, int max_kv_len,
                              int num_heads, int num_kv_heads, int head_dim, int block_size,
                              int64_t num_blocks, float scale, int dtype, int splits,
                              void* workspace, size_t workspace_bytes, void* stream);
int mvllm_prefill_paged_int8_split(void* out, const void* q,
                                   const int8_t* k_cache, const int8_t* v_cache,
                                   const float* k_scale, const float* v_scale,
                                   const int32_t* block_tables, int max_num_blocks,
                                   const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                   int num_seqs, int64_t total_q_tokens, int max_kv_len,
                                   int num_heads, int num_kv_heads, int head_dim, int block_size,
                                   int64_t num_blocks, float scale, int dtype, int splits,
                                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * The caller's per-layer chain between the QKV projection and the attention kernels, fused:
 *   q = rms_norm(q); k = rms_norm(k)      src/myvllm/models/qwen3.py:104-106, layers/layernorm.py:9-17
 *   q, k = rotary_emb(positions, q, k)    qwen3.py:108, layers/rotary_embedding.py:4-23, 77-83
 *   store_kvcache(k, v, ...)              layers/attention.py:67-108 (called from Attention.forward :505-506)
 * q, k, v are rows of num_heads*D / num_kv_heads*D / num_kv_heads*D elements with the given strides (in
 * elements) between tokens, so the three slices of the packed QKV projection output can be passed as they
 * lie.  gamma [D] fp32 is the shared RMSNorm weight (NULL: no norm, the reference's qkv_bias=True case);
 * cos_sin_cache [max_position, D] fp32 holds cos (D/2) then sin (D/2) per position (rotary_embedding.py:61-70);
 * positions int64 [T] are clamped to [0, max_position).  Rotation pairs element i with i + D/2.
 * Rounding follows the unfused chain: norm result rounded to the element type, rotation in fp32 on the
 * rounded values, rounded again.
 * Outputs: q_out [T, Hq, D] always; k_out / v_out [T, Hkv, D] when not NULL (the prefill kernel reads them);
 * when slot_mapping is not NULL the rotated k and v go to flat slot slot_mapping[t] of the caches
 * (slots < 0 or >= num_slots skipped): element-type caches, or with cache_is_int8 != 0 int8 codes and
 * fp32 scales exactly as mvllm_store_kvcache_int8 would write them from k_out / v.
 * head_dim % 8 == 0, head_dim <= 512; 8-byte aligned pointers (16-byte for fp32), strides % 4 == 0.
 */
int mvllm_qk_norm_rope_store(void* q_out, void* k_out, void* v_out,
                             const void* q, const void* k, const void* v,
                             int64_t q_row_stride, int64_t k_row_stride, int64_t v_row_stride,
                             const float* gamma, float eps,
                             const float* cos_sin_cache, int64_t max_position,
                             const int64_t* positions, const int64_t* slot_mapping,
                             void* k_cache, void* v_cache, float* k_scale, float* v_scale, int cache_is_int8,
                             int64_t num_tokens, int64_t num_slots,
                             int num_heads, int num_kv_heads, int head_dim, int dtype, void* stream);

/*
 * SamplerLayer.forward -- src/myvllm/layers/sampler.py:14-19:
 *   logits /= temperature; probs = softmax(logits); token = argmax(probs / exponential_(1).clamp_min_(1e-10))
 * One launch, no (batch, vocab) probability tensor: out_ids[b] = argmax_i( logits[b,i] / temperatures[b]
 * - log(max(E[b,i], 1e-10)) ), which is the same argmax (softmax only rescales a row by a positive factor).
 * Ties go to the smallest index.
 *   logits        [batch, vocab] in dtype, row_stride elements between rows (the LM-head GEMM output as it lies)
 *   temperatures  fp32 [batch], > 0
 *   noise         fp32 [batch, vocab] of Exp(1) draws, or NULL: then E comes from Philox4x32-10 with key = seed
 *                 and counter = (i / 4, b, offset): lane (i % 4) of the output word gives u = ((x >> 8) + 0.5) * 2^-24
 *                 and E = -log(u).  Advance `offset` by one per call for independent draws.
 *   out_ids       int64 [batch]
 *   workspace     optional scratch of mvllm_sample_tokens_workspace_bytes(batch, vocab) bytes: with it a row is
 *                 scanned by several workgroups (a small batch alone cannot occupy the GPU) and a second tiny
 *                 launch picks the winner; NULL or too small: one workgroup per row, same result.
 */
size_t mvllm_sample_tokens_workspace_bytes(int batch, int vocab);
int mvllm_sample_tokens(int64_t* out_ids, const void* logits, int64_t row_stride,
                        const float* temperatures, const float* noise,
                        uint64_t seed, uint64_t offset, int batch, int vocab, int dtype,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * mvllm_sample_tokens with in-kernel noise whose call offset is read from device memory (*offset_dev), for a
 * sampler inside a captured graph: a replay cannot change a launch argument, the graph increments the counter.
 */
int mvllm_sample_tokens_dev_offset(int64_t* out_ids, const void* logits, int64_t row_stride,
                                   const float* temperatures, uint64_t seed, const uint64_t* offset_dev,
                                   int batch, int vocab, int dtype,
                                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * LM head + sampler in one pass over the weights -- ParallelLMHead.forward (src/myvllm/layers/embedding_head.py:56-77:
 * rows to sample from, hidden W^T) followed by SamplerLayer.forward (layers/sampler.py:14-19), without the
 * (batch, vocab) logits reaching memory:
 *   out_ids[b] = argmax_n( bf16(hidden[row_index[b]] . W[n]) / T[b] - log(max(E[b, n], 1e-10)) )
 * with the logit rounded to the element type, as the materialised tensor would be, and E drawn as in
 * mvllm_sample_tokens (Philox4x32-10, key = seed, counter = (n / 4, b, offset (+ *offset_dev when not NULL))): the
 * same ids as mvllm_sample_tokens on the rounded product, up to the order of the fp32 sums inside a logit.
 * hidden rows hidden_row_stride elements apart (a multiple of 8); row_index int64 [batch] or NULL (rows 0..batch-1:
 * a decode step; the last token of every packed sequence in prefill, embedding_head.py:57-62); weight [vocab, K]
 * dense.  batch <= 64, vocab % 16 == 0, K in {256, 512, 1024}, bf16 / fp16; otherwise MVLLM_ERR_UNSUPPORTED and the
 * caller runs the library GEMM and mvllm_sample_tokens.  workspace: mvllm_lm_head_sample_workspace_bytes(batch, K)
 * bytes, 8-byte aligned, caller-owned.  The first launch of a shape with more than 48 KB of hidden rows raises the
 * kernel's dynamic LDS limit (a host-side attribute call: make it outside a graph capture).
 */
size_t mvllm_lm_head_sample_workspace_bytes(int batch, int K);
int mvllm_lm_head_sample(int64_t* out_ids, const void* hidden, int64_t hidden_row_stride,
                         const int64_t* row_index, const void* weight, const float* temperatures,
                         uint64_t seed, uint64_t offset, const uint64_t* offset_dev, int batch, int vocab,
                         int K, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The step metadata of a decode batch that continues the step before it (same sequences, each one token longer),
 * advanced on the device in one launch instead of being rebuilt on the host as ModelRunner.prepare_decode does
 * (src/myvllm/engine/model_runner.py:231-256): input_ids[i] = sampled[i]; context_lens[i] += 1;
 * positions[i] = context_lens[i] - 1; slot_mapping[i] += 1.  All int64 [batch].  Rows whose context length is
 * not positive (the padding of a captured batch size) are left alone.  Rows that open a new block have their slot
 * and table entry patched by the caller afterwards.  step_counter (may be NULL): one uint64 on the device, the
 * call counter of mvllm_sample_tokens_dev_offset / mvllm_lm_head_sample, incremented by one, so that a captured
 * decode step can end with this launch and be replayed without any host-side update.  host_ids (may be NULL; needs
 * step_counter): two rows of host_row_stride >= batch + 1 int64 in pinned, device-visible host memory; row
 * (counter before the increment) & 1 receives sampled[0 .. batch) and then, behind a system-scope fence, the new
 * counter value in its last entry: the host reads a step's ids once it sees that value, with no copy operation and
 * no event queued between two replays (two rows: step t is read while step t + 1 runs).
 */
int mvllm_decode_advance(int64_t* input_ids, int64_t* context_lens, int64_t* positions, int64_t* slot_mapping,
                         const int64_t* sampled, uint64_t* step_counter, int64_t* host_ids,
                         int64_t host_row_stride, int batch, void* stream);

/*
 * LayerNorm.forward with and without residual -- src/myvllm/layers/layernorm.py:9-28, called from
 * Qwen3DecoderLayer.forward and the final norm (src/myvllm/models/qwen3.py:197-212, 306-312):
 *   x = x + residual (rounded to the element type);  out = x / sqrt(mean(x^2) + eps) * gamma;  residual_out = x
 * x [rows, hidden] with x_row_stride elements between rows; residual likewise or NULL (no add);
 * residual_out [rows, hidden] dense or NULL; out [rows, hidden] dense; gamma fp32 [hidden].
 * hidden % 8 == 0, hidden <= 8192, 16-byte aligned pointers, strides % 8 == 0.
 */
int mvllm_add_rms_norm(void* out, void* residual_out, const void* x, const void* residual,
                       const float* gamma, float eps, int64_t rows, int hidden,
                       int64_t x_row_stride, int64_t residual_row_stride, int dtype, void* stream);

/*
 * SiluAndMul.forward -- src/myvllm/layers/activation.py:15-18:  x, y = in.chunk(2, -1); out = silu(x) * y
 * in [rows, 2*width] with in_row_stride elements between rows; out [rows, width] dense.  silu(x) is rounded to
 * the element type before the product, as the two tensor operations would.  width a multiple of 16 bytes.
 */
int mvllm_silu_and_mul(void* out, const void* in, int64_t rows, int width, int64_t in_row_stride,
                       int dtype, void* stream);

/*
 * The caller's projections around the attention path for the few rows of a decode step -- nn.Linear in
 * src/myvllm/models/qwen3.py:90-94 (QKV), :118 (output projection) and the MLP (:121-160; layers/linear.py):
 *   out[M, N] = x[M, K] W[N, K]^T + bias[N]
 * M <= 64, bf16 / fp16 with fp32 accumulation, N % 16 == 0, K % 512 == 0; x rows x_row_stride elements apart
 * (a multiple of 8), W dense, bias in the element type or NULL; x and W 16-byte aligned.  Larger M (prefill) stays
 * a library GEMM: MVLLM_ERR_UNSUPPORTED.
 */
int mvllm_linear_small_m(void* out, const void* x, const void* w, const void* bias, int64_t x_row_stride,
                         int M, int N, int K, int dtype, void* stream);

/*
 * The same product with the launches around it folded in, for the decoder layer's decode step
 * (src/myvllm/models/qwen3.py:197-212: residual add + RMSNorm, projection; :151-160: gate/up, SiluAndMul):
 *   gamma != NULL:  h = x + residual (rounded to the element type; residual NULL: h = x), residual_out = h (may be
 *                   NULL), x' = h / sqrt(mean(h^2) + eps) * gamma rounded to the element type, exactly what
 *                   mvllm_add_rms_norm writes (layers/layernorm.py:9-28) up to the order of the sum of squares;
 *                   the product is taken of x'.  residual and residual_out are dense [M, K]; residual_out must not
 *                   alias x or residual (every workgroup reads all of both while one of them writes a row).
 *   glu != 0:       W is [2F, K] (gate rows, then up rows, as layers/activation.py:15-18 chunks the output), out is
 *                   [M, F] = silu(x' Wg^T + bg) * (x' Wu^T + bu) with the roundings of mvllm_silu_and_mul on the
 *                   rounded projection; N = 2F, N % 32 == 0.
 * Shapes as mvllm_linear_small_m, and for gamma != NULL: N / 16 >= min(M, 16), K / waves one burst of 128 or 256
 * values with 4, 8 or 16 waves (mvllm_linear_small_m_plan says whether a shape is taken); otherwise MVLLM_ERR_UNSUPPORTED and the caller
 * runs the separate launches.
 */
int mvllm_norm_linear_small_m(void* out, void* residual_out, const void* x, const void* residual,
                              const float* gamma, float eps, const void* w, const void* bias,
                              int64_t x_row_stride, int M, int N, int K, int glu, int dtype, void* stream);

/*
 * Whether mvllm_linear_small_m (norm == 0 && glu == 0) or mvllm_norm_linear_small_m takes a shape, without a
 * launch: MVLLM_OK and the waves per workgroup in *waves (may be NULL), or MVLLM_ERR_UNSUPPORTED.  No counterpart
 * in the reference (its projections are library GEMMs of any shape).
 */
int mvllm_linear_small_m_plan(int M, int N, int K, int norm, int glu, int dtype, int* waves);

#ifdef __cplusplus
}
#endif
#endif /* MINIVLLM_AMD_H_ */
