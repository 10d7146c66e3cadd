"""CPU restatement (torch-CPU / numpy) of the reference's attention path.

TEST INFRASTRUCTURE ONLY: imported by tests/, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.  The product package never imports it.

Each function names the reference lines whose algorithm it restates.  The
reference has no tests or golden vectors for this path, so each function is
pinned by ``tests/test_oracle_pins.py`` against what the mathematics fixes:

* ``store_kvcache_oracle``      closed form on a poison-filled cache, round trip
* ``decode_naive_oracle``       fp64 brute force, ctx=1, equal-K mean, dense SDPA
* ``decode_vectorised_oracle``  same checks + equality with the naive one
* ``prefill_standard_oracle``   per-sequence ``scaled_dot_product_attention``
                                (library routine), row-0 identity, fp64 brute force
* ``quantize_int8_oracle``      spec invariants (|code|<=127, max|code|==127,
                                |x-code*scale|<=scale/2, scale == amax/127 in fp32)
                                -- "parity unpinned" by the reference: it has no
                                INT8 code; the spec is defined by this build.
* ``prefill_paged_oracle``       equals the last rows of ``prefill_standard_oracle`` on the
                                full sequences; no cached prefix == plain prefill; one
                                new token == the decode oracle
* ``rms_norm_oracle`` / ``rope_cos_sin_cache_oracle`` / ``rope_oracle`` /
  ``qk_norm_rope_store_oracle``   unit mean square, scale invariance, constant-vector
                                closed form; table vs cos/sin of pos * base^(-2i/D) in
                                fp64; position 0 identity, hand-worked quarter turn
                                (sign and half-split pairing), pair norms kept,
                                angles add, scores depend on position difference only
"""
from __future__ import annotations

import torch


# --------------------------------------------------------------------------
# store_kvcache        reference: src/myvllm/layers/attention.py:25-64, 67-108
# --------------------------------------------------------------------------
def store_kvcache_oracle(key, value, k_cache, v_cache, slot_mapping, block_size):
    """Scatter token rows into the flat slot view of the paged caches.

    The reference kernel splits a slot into (block, offset) and re-multiplies
    by block_size (attention.py:33-34, 53-56); for a contiguous
    ``[num_blocks, block_size, Hkv, D]`` cache that is the flat row ``slot``.
    Rows whose slot is -1 are skipped (attention.py:29-30).
    """
    num_tokens, num_kv_heads, head_dim = key.shape
    assert k_cache.shape == v_cache.shape          # attention.py:94
    assert slot_mapping.numel() == num_tokens      # attention.py:95
    flat_k = k_cache.view(-1, num_kv_heads, head_dim)
    flat_v = v_cache.view(-1, num_kv_heads, head_dim)
    slots = slot_mapping.to(torch.int64).tolist()
    for t, slot in enumerate(slots):
        if slot == -1:
            continue
        flat_k[slot] = key[t]
        flat_v[slot] = value[t]


# --------------------------------------------------------------------------
# INT8 KV-cache spec (no reference symbol; defined by this build)
# --------------------------------------------------------------------------
def quantize_int8_oracle(x: torch.Tensor):
    """Per (token, head) symmetric INT8 quantisation.

    amax = max|x| over head_dim in fp32; scale = amax / 127 (IEEE fp32 divide);
    code = clamp(round_half_even(x / scale), -127, 127); amax == 0 gives
    scale 0 and codes 0.  Returns (codes int8 [..., D], scales fp32 [...]).
    """
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=-1)
    scale = amax / torch.tensor(127.0, dtype=torch.float32)
    safe = torch.where(scale > 0, scale, torch.ones_like(scale))
    codes = torch.round(xf / safe.unsqueeze(-1)).clamp_(-127.0, 127.0)
    codes = torch.where(scale.unsqueeze(-1) > 0, codes, torch.zeros_like(codes))
    return codes.to(torch.int8), scale


def store_kvcache_int8_oracle(key, value, k_cache, v_cache, k_scale, v_scale,
                              slot_mapping, block_size):
    """Quantise then scatter codes and scales with the store_kvcache rule."""
    num_tokens, num_kv_heads, head_dim = key.shape
    assert k_cache.shape == v_cache.shape
    assert slot_mapping.numel() == num_tokens
    kc, ks = quantize_int8_oracle(key)
    vc, vs = quantize_int8_oracle(value)
    flat_k = k_cache.view(-1, num_kv_heads, head_dim)
    flat_v = v_cache.view(-1, num_kv_heads, head_dim)
    flat_ks = k_scale.view(-1, num_kv_heads)
    flat_vs = v_scale.view(-1, num_kv_heads)
    for t, slot in enumerate(slot_mapping.to(torch.int64).tolist()):
        if slot == -1:
            continue
        flat_k[slot] = kc[t]
        flat_v[slot] = vc[t]
        flat_ks[slot] = ks[t]
        flat_vs[slot] = vs[t]


def dequantize_cache_oracle(codes: torch.Tensor, scales: torch.Tensor):
    """fp32 cache ``code * scale`` from int8 codes [NB,bs,Hkv,D], scales [NB,bs,Hkv]."""
    return codes.to(torch.float32) * scales.to(torch.float32).unsqueeze(-1)


# --------------------------------------------------------------------------
# paged decode         reference: benchmark_decoding.py:192-269 (naive),
#                                 benchmark_decoding.py:136-189 (vectorised)
# --------------------------------------------------------------------------
def gather_sequence_kv(cache, table_row, seq_len, block_size):
    """Rows 0..seq_len-1 of one sequence in logical order.

    benchmark_decoding.py:221-233: walk the first ceil(seq_len/bs) table
    entries, concatenate whole blocks, truncate to seq_len.
    """
    need = (seq_len + block_size - 1) // block_size
    ids = [int(b) for b in table_row[:need].tolist()]
    blocks = [cache[b] for b in ids]
    return torch.cat(blocks, dim=0)[:seq_len]


def _padded_softmax_attention(q, padded_k, padded_v, context_lens, scale,
                              num_heads, num_kv_heads):
    """Shared tail of both reference decode functions.

    benchmark_decoding.py:248-269 == :171-189: repeat KV heads for GQA,
    (B,H,1,D)x(B,H,D,N) scores * scale, mask positions >= context_len with
    -inf, softmax, times V.
    """
    if num_kv_heads != num_heads:
        rep = num_heads // num_kv_heads
        padded_k = padded_k.repeat_interleave(rep, dim=2)
        padded_v = padded_v.repeat_interleave(rep, dim=2)
    max_len = padded_k.shape[1]
    qh = q.unsqueeze(2)                                   # (B,H,1,D)
    kh = padded_k.permute(0, 2, 3, 1)                     # (B,H,D,N)
    vh = padded_v.permute(0, 2, 1, 3)                     # (B,H,N,D)
    scores = torch.matmul(qh, kh) * scale                 # (B,H,1,N)
    live = torch.arange(max_len)[None, :] < context_lens.to(torch.int64)[:, None]
    scores = scores.masked_fill(~live[:, None, None, :], float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.matmul(probs, vh).squeeze(2)             # (B,H,D)


def decode_naive_oracle(q, k_cache, v_cache, block_tables, context_lens, scale,
                        num_heads, num_kv_heads, head_dim, block_size):
    """benchmark_decoding.py:192-269: per-sequence gather by block table,
    zero-pad to the longest context, one masked softmax attention.

    Valid inputs only (every needed table entry >= 0, context_len >= 1); the
    reference's behaviour on -1 entries inside the needed range or on
    context_len 0 (NaN) is not reproduced.
    """
    batch = q.shape[0]
    lens = [int(x) for x in context_lens.tolist()]
    max_len = max(lens)
    padded_k = torch.zeros(batch, max_len, num_kv_heads, head_dim, dtype=q.dtype)
    padded_v = torch.zeros_like(padded_k)
    for b, n in enumerate(lens):
        padded_k[b, :n] = gather_sequence_kv(k_cache, block_tables[b], n, block_size).to(q.dtype)
        padded_v[b, :n] = gather_sequence_kv(v_cache, block_tables[b], n, block_size).to(q.dtype)
    return _padded_softmax_attention(q, padded_k, padded_v, context_lens, scale,
                                     num_heads, num_kv_heads)


def decode_vectorised_oracle(q, k_cache, v_cache, block_tables, context_lens, scale,
                             num_heads, num_kv_heads, head_dim, block_size):
    """benchmark_decoding.py:136-189: same result, gathering each sequence's
    blocks with one fancy-index instead of a Python loop over blocks."""
    batch = q.shape[0]
    lens = [int(x) for x in context_lens.tolist()]
    max_len = max(lens)
    padded_k = torch.zeros(batch, max_len, num_kv_heads, head_dim, dtype=q.dtype)
    padded_v = torch.zeros_like(padded_k)
    for b, n in enumerate(lens):
        need = (n + block_size - 1) // block_size
        ids = block_tables[b, :need].to(torch.int64)
        ids = ids[ids != -1]
        if ids.numel() == 0:
            continue
        padded_k[b, :n] = k_cache[ids].reshape(-1, num_kv_heads, head_dim)[:n].to(q.dtype)
        padded_v[b, :n] = v_cache[ids].reshape(-1, num_kv_heads, head_dim)[:n].to(q.dtype)
    return _padded_softmax_attention(q, padded_k, padded_v, context_lens, scale,
                                     num_heads, num_kv_heads)


def decode_int8_oracle(q, k_codes, v_codes, k_scale, v_scale, block_tables, context_lens,
                       scale, num_heads, num_kv_heads, head_dim, block_size):
    """INT8 decode spec: dequantise (code*scale in fp32) then the naive decode."""
    kf = dequantize_cache_oracle(k_codes, k_scale)
    vf = dequantize_cache_oracle(v_codes, v_scale)
    return decode_naive_oracle(q.to(torch.float32), kf, vf, block_tables, context_lens,
                               scale, num_heads, num_kv_heads, head_dim, block_size)


# --------------------------------------------------------------------------
# varlen causal prefill    reference: benchmark_prefilling.py:9-52
# --------------------------------------------------------------------------
def prefill_standard_oracle(q, k, v, cu_seqlens, scale, num_heads, num_kv_heads, head_dim):
    """benchmark_prefilling.py:9-52: for every packed sequence, heads-major
    (H,L,D), repeat KV heads for GQA, full L x L scores * scale, strictly upper
    triangle masked to -inf, softmax, times V; rows written back packed."""
    out = torch.zeros_like(q)
    bounds = [int(x) for x in cu_seqlens.tolist()]
    for s in range(len(bounds) - 1):
        lo, hi = bounds[s], bounds[s + 1]
        n = hi - lo
        if n == 0:
            continue
        qs = q[lo:hi].transpose(0, 1)
        ks = k[lo:hi].transpose(0, 1)
        vs = v[lo:hi].transpose(0, 1)
        if num_kv_heads != num_heads:
            rep = num_heads // num_kv_heads
            ks = ks.repeat_interleave(rep, dim=0)
            vs = vs.repeat_interleave(rep, dim=0)
        scores = torch.matmul(qs, ks.transpose(1, 2)) * scale
        future = torch.ones(n, n, dtype=torch.bool).triu(diagonal=1)
        scores = scores.masked_fill(future.unsqueeze(0), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[lo:hi] = torch.matmul(probs, vs).transpose(0, 1)
    return out


def prefill_paged_oracle(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k, scale,
                         num_heads, num_kv_heads, head_dim, block_size):
    """Prefill of the tokens after a cached prefix: what ``pytorch_standard_attention``
    (benchmark_prefilling.py:9-52) gives for the LAST len_q rows of each sequence when its keys are gathered
    from the paged cache in logical order (``gather_sequence_kv``, benchmark_decoding.py:228-233) --
    the computation the metadata of model_runner.py:192-226 describes.  fp32 math, result in q's dtype."""
    out = torch.empty_like(q)
    group = num_heads // num_kv_heads
    cq, ck = cu_seqlens_q.tolist(), cu_seqlens_k.tolist()
    for s in range(len(cq) - 1):
        lq, lk = cq[s + 1] - cq[s], ck[s + 1] - ck[s]
        if lq == 0:
            continue
        cached = lk - lq
        k = gather_sequence_kv(k_cache, block_tables[s], lk, block_size).float()
        v = gather_sequence_kv(v_cache, block_tables[s], lk, block_size).float()
        k = k.repeat_interleave(group, dim=1).transpose(0, 1)                 # (Hq, lk, D)
        v = v.repeat_interleave(group, dim=1).transpose(0, 1)
        qs = q[cq[s]:cq[s + 1]].float().transpose(0, 1)                       # (Hq, lq, D)
        scores = torch.matmul(qs, k.transpose(1, 2)) * scale                  # (Hq, lq, lk)
        pos = torch.arange(lq).unsqueeze(1) + cached                          # key j visible iff j <= cached + i
        scores = scores.masked_fill(torch.arange(lk).unsqueeze(0) > pos, float("-inf"))
        out[cq[s]:cq[s + 1]] = torch.matmul(torch.softmax(scores, dim=-1), v).transpose(0, 1).to(q.dtype)
    return out


# --------------------------------------------------------------------------
# caller-side chain in front of the attention kernels
# reference: src/myvllm/models/qwen3.py:104-110, layers/layernorm.py:9-17,
#            layers/rotary_embedding.py:4-23 and :48-83, layers/attention.py:505-506
# --------------------------------------------------------------------------
def rms_norm_oracle(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * gamma over the last dim, fp32 math, result in x's dtype
    (layernorm.py:13-15)."""
    xf = x.float()
    variance = xf.pow(2).mean(dim=-1, keepdim=True) + eps
    return (xf / variance.sqrt() * gamma.float()).to(x.dtype)


def rope_cos_sin_cache_oracle(base: float, rotary_dim: int, max_position: int) -> torch.Tensor:
    """[max_position, rotary_dim] fp32: cos(pos * inv_freq) | sin(pos * inv_freq),
    inv_freq[i] = base^(-2i/rotary_dim) (rotary_embedding.py:58-70)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    freqs = torch.einsum("i,j->ij", torch.arange(max_position, dtype=torch.float32), inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1)


def rope_oracle(x: torch.Tensor, positions: torch.Tensor, cos_sin_cache: torch.Tensor) -> torch.Tensor:
    """Half-split rotation of x (T, H, D): element i pairs with i + D/2
    (rotary_embedding.py:4-23, 77-83).  fp32 math, result in x's dtype."""
    cos, sin = cos_sin_cache[positions.long()].float().chunk(2, dim=-1)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    x1, x2 = x.float().chunk(2, dim=-1)
    return torch.cat([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).to(x.dtype)


def qk_norm_rope_store_oracle(q, k, v, positions, cos_sin_cache, gamma, eps, slot_mapping=None,
                              k_cache=None, v_cache=None, k_scale=None, v_scale=None, block_size=0):
    """The unfused chain: shared-gamma RMSNorm on q and k (skipped when gamma is None, the
    reference's qkv_bias=True case), rotation, then the cache store of (rotated k, v).
    Returns (q_out, k_out); caches are modified in place (int8 when k_scale is given)."""
    if gamma is not None:
        q, k = rms_norm_oracle(q, gamma, eps), rms_norm_oracle(k, gamma, eps)
    q, k = rope_oracle(q, positions, cos_sin_cache), rope_oracle(k, positions, cos_sin_cache)
    if slot_mapping is not None:
        if k_scale is not None:
            store_kvcache_int8_oracle(k, v, k_cache, v_cache, k_scale, v_scale, slot_mapping, block_size)
        else:
            store_kvcache_oracle(k, v, k_cache, v_cache, slot_mapping, block_size)
    return q, k


def add_rms_norm_oracle(x, gamma, eps, residual=None):
    """LayerNorm.forward (layernorm.py:19-28): with a residual the sum is formed (and rounded) in x's dtype,
    normalised, and returned next to the sum."""
    if residual is None:
        return rms_norm_oracle(x, gamma, eps)
    s = x + residual
    return rms_norm_oracle(s, gamma, eps), s


def silu_and_mul_oracle(x):
    """SiluAndMul.forward (activation.py:15-18) as two tensor operations: silu in fp32 rounded to x's dtype,
    then the product rounded again."""
    a, b = x.chunk(2, dim=-1)
    af = a.float()
    s = (af / (1.0 + torch.exp(-af))).to(x.dtype)
    return (s.float() * b.float()).to(x.dtype)
