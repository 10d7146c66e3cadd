"""Fused caller-side operator in front of the attention kernels.

``qk_norm_rope_store`` does in one HIP launch what the reference's ``Qwen3Attention.forward`` does with
three modules per layer and step (src/myvllm/models/qwen3.py:104-110): the shared-gamma RMSNorm of q and k
(layers/layernorm.py:9-17), the half-split rotary embedding (layers/rotary_embedding.py:4-23, 77-83) and
``store_kvcache`` of the rotated k and of v (layers/attention.py:67-108).  It reads q, k and v as the three
column slices of the packed QKV projection output (no copies) and calls libminivllm_amd.so on the current
torch stream; there is no PyTorch fallback.

``sample_tokens`` is the reference's ``SamplerLayer.forward`` (layers/sampler.py:14-19) as one launch over the
LM-head output, with the Exp(1) noise drawn inside the kernel (Philox4x32-10) or passed in.
"""
from __future__ import annotations

import torch

from minivllm_amd import _C

__all__ = ["qk_norm_rope_store", "sample_tokens", "sample_tokens_into", "decode_advance", "add_rms_norm", "silu_and_mul", "linear_small_m", "linear_small_m_takes", "norm_linear_small_m", "norm_linear_small_m_takes",
           "lm_head_sample", "lm_head_sample_takes", "lm_head_sample_workspace_bytes"]


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _rows(name, t, heads, head_dim):
    """(T, heads, head_dim) view whose (head, dim) part is dense; returns the token stride in elements."""
    if t.dim() != 3 or tuple(t.shape[1:]) != (heads, head_dim):
        raise ValueError(f"{name} must be (num_tokens, {heads}, {head_dim}), got {tuple(t.shape)}")
    if t.shape[0] > 1 and (t.stride(2) != 1 or t.stride(1) != head_dim):
        raise ValueError(f"{name}: heads and head_dim must be contiguous inside a token row")
    return t.stride(0) if t.shape[0] > 1 else heads * head_dim


def qk_norm_rope_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
                       cos_sin_cache: torch.Tensor, gamma: torch.Tensor | None = None, eps: float = 1e-6,
                       slot_mapping: torch.Tensor | None = None, k_cache: torch.Tensor | None = None,
                       v_cache: torch.Tensor | None = None, k_scale: torch.Tensor | None = None,
                       v_scale: torch.Tensor | None = None, need_kv: bool = True):
    """RMSNorm(q), RMSNorm(k) with one gamma over head_dim (skipped when ``gamma`` is None), rotary embedding
    of both at ``positions``, and the cache store of the rotated k and of v at ``slot_mapping``.

    q: (T, Hq, D); k, v: (T, Hkv, D), token rows may be strided (slices of the QKV projection);
    positions int64 (T,); cos_sin_cache float32 (max_position, D) = cos | sin; gamma float32 (D,);
    caches (num_blocks, block_size, Hkv, D) in q's dtype, or int8 with float32 k_scale / v_scale
    (num_blocks, block_size, Hkv).  ``slot_mapping`` None stores nothing.
    Returns (q_out, k_out, v_out) contiguous; k_out and v_out are None unless ``need_kv`` (prefill reads
    them, decode reads the cache).
    """
    _C.require_cuda(q, k, v, positions, cos_sin_cache)
    if q.dim() != 3 or k.dim() != 3:
        raise ValueError("q, k and v must be (num_tokens, heads, head_dim)")
    num_tokens, num_heads, head_dim = q.shape
    num_kv_heads = k.shape[1]
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k and v must share one dtype")
    if k.shape[0] != num_tokens or v.shape != k.shape:
        raise ValueError("q, k and v must have the same number of tokens and k, v the same shape")
    q_stride = _rows("q", q, num_heads, head_dim)
    k_stride = _rows("k", k, num_kv_heads, head_dim)
    v_stride = _rows("v", v, num_kv_heads, head_dim)
    if positions.numel() != num_tokens:
        raise ValueError("positions must have one entry per token")
    if positions.dtype != torch.int64:
        positions = positions.to(torch.int64)
    positions = positions.contiguous()
    if cos_sin_cache.dtype != torch.float32 or cos_sin_cache.dim() != 2 or cos_sin_cache.shape[1] != head_dim \
            or not cos_sin_cache.is_contiguous():
        raise ValueError(f"cos_sin_cache must be contiguous float32 (max_position, {head_dim})")
    if gamma is not None:
        _C.require_cuda(gamma)
        if gamma.dtype != torch.float32 or gamma.numel() != head_dim or not gamma.is_contiguous():
            raise ValueError(f"gamma must be contiguous float32 ({head_dim},)")
    int8 = False
    num_slots = 0
    if slot_mapping is not None:
        if k_cache is None or v_cache is None:
            raise ValueError("slot_mapping given without caches")
        _C.require_cuda(slot_mapping, k_cache, v_cache)
        if slot_mapping.numel() != num_tokens:
            raise ValueError("Slot mapping size must match number of tokens")
        if slot_mapping.dtype != torch.int64:
            slot_mapping = slot_mapping.to(torch.int64)
        slot_mapping = slot_mapping.contiguous()
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dim() != 4 or tuple(c.shape[2:]) != (num_kv_heads, head_dim) or not c.is_contiguous():
                raise ValueError(f"{name} must be contiguous [num_blocks, block_size, {num_kv_heads}, {head_dim}]")
        if k_cache.shape != v_cache.shape:
            raise ValueError("K and V cache shapes must match")
        int8 = k_cache.dtype == torch.int8
        if int8:
            if v_cache.dtype != torch.int8:
                raise ValueError("int8 caches expected")
            for name, s in (("k_scale", k_scale), ("v_scale", v_scale)):
                if s is None or s.dtype != torch.float32 or tuple(s.shape) != tuple(k_cache.shape[:3]) \
                        or not s.is_contiguous():
                    raise ValueError(f"{name} must be contiguous float32 {tuple(k_cache.shape[:3])}")
        elif k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
            raise ValueError(f"cache dtype {k_cache.dtype} differs from q/k/v dtype {q.dtype}")
        num_slots = k_cache.shape[0] * k_cache.shape[1]
    q_out = torch.empty((num_tokens, num_heads, head_dim), dtype=q.dtype, device=q.device)
    k_out = torch.empty((num_tokens, num_kv_heads, head_dim), dtype=q.dtype, device=q.device) if need_kv else None
    v_out = torch.empty_like(k_out) if need_kv else None
    if num_tokens == 0:
        return q_out, k_out, v_out
    lib = _C.load()
    st = lib.mvllm_qk_norm_rope_store(
        _ptr(q_out), _ptr(k_out), _ptr(v_out), _ptr(q), _ptr(k), _ptr(v), q_stride, k_stride, v_stride,
        _ptr(gamma), float(eps), _ptr(cos_sin_cache), cos_sin_cache.shape[0], _ptr(positions),
        _ptr(slot_mapping), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale if int8 else None),
        _ptr(v_scale if int8 else None), int(int8), num_tokens, num_slots, num_heads, num_kv_heads, head_dim,
        _C.dtype_code(q.dtype), _C.current_stream_ptr(q.device))
    _C.check(st, "qk_norm_rope_store")
    return q_out, k_out, v_out


def sample_tokens(logits: torch.Tensor, temperatures: torch.Tensor, seed: int = 0, offset: int = 0,
                  noise: torch.Tensor | None = None, use_workspace: bool = True) -> torch.Tensor:
    """One token per row from softmax(logits / temperature): argmax of ``probs / Exp(1) noise`` as in
    sampler.py:15-18, computed as argmax(logits / T - log(noise)) without a probability tensor.

    logits: (batch, vocab) float32 / bfloat16 / float16, rows may be strided; temperatures float32 (batch,), > 0.
    ``noise`` float32 (batch, vocab) supplies the draws (clamped below at 1e-10); without it they are generated
    from (seed, offset): the same pair always gives the same tokens, advance ``offset`` per call.
    ``use_workspace=False`` keeps every row in one workgroup (same tokens, slower for small batches).
    Returns int64 (batch,).
    """
    _C.require_cuda(logits, temperatures, noise)
    if logits.dim() != 2:
        raise ValueError(f"logits must be (batch, vocab), got {tuple(logits.shape)}")
    batch, vocab = logits.shape
    if batch > 1 and logits.stride(1) != 1 or batch == 1 and vocab > 1 and logits.stride(1) != 1:
        logits = logits.contiguous()
    if temperatures.numel() != batch:
        raise ValueError("temperatures must have one entry per row")
    temperatures = temperatures.to(torch.float32).contiguous()
    if noise is not None:
        if tuple(noise.shape) != (batch, vocab) or noise.dtype != torch.float32:
            raise ValueError(f"noise must be float32 ({batch}, {vocab})")
        noise = noise.contiguous()
    out = torch.empty(batch, dtype=torch.int64, device=logits.device)
    if batch == 0:
        return out
    lib = _C.load()
    nbytes = lib.mvllm_sample_tokens_workspace_bytes(batch, vocab) if use_workspace else 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=logits.device) if nbytes else None
    st = lib.mvllm_sample_tokens(_ptr(out), _ptr(logits), logits.stride(0) if batch > 1 else vocab,
                                 _ptr(temperatures), _ptr(noise), int(seed) & (2 ** 64 - 1),
                                 int(offset) & (2 ** 64 - 1), batch, vocab, _C.dtype_code(logits.dtype),
                                 _ptr(ws), nbytes, _C.current_stream_ptr(logits.device))
    _C.check(st, "sample_tokens")
    return out


def sample_tokens_into(out: torch.Tensor, logits: torch.Tensor, temperatures: torch.Tensor, seed: int,
                       offset_dev: torch.Tensor, workspace: torch.Tensor | None) -> None:
    """``sample_tokens`` for a captured graph: nothing is allocated (``out`` int64 (batch,), ``workspace`` uint8 from
    ``sample_workspace_bytes`` or None) and the call offset is read from ``offset_dev`` (one uint64 / int64 on the
    device, which the graph increments), so every replay draws fresh noise."""
    _C.require_cuda(out, logits, temperatures, offset_dev, workspace)
    batch, vocab = logits.shape
    if logits.stride(1) != 1 or out.numel() != batch or out.dtype != torch.int64 or temperatures.dtype != torch.float32:
        raise ValueError("logits rows must be dense, out int64 (batch,), temperatures float32 (batch,)")
    st = _C.load().mvllm_sample_tokens_dev_offset(
        _ptr(out), _ptr(logits), logits.stride(0) if batch > 1 else vocab, _ptr(temperatures),
        int(seed) & (2 ** 64 - 1), _ptr(offset_dev), batch, vocab, _C.dtype_code(logits.dtype), _ptr(workspace),
        0 if workspace is None else workspace.numel(), _C.current_stream_ptr(logits.device))
    _C.check(st, "sample_tokens_into")


def sample_workspace_bytes(batch: int, vocab: int) -> int:
    return int(_C.load().mvllm_sample_tokens_workspace_bytes(batch, vocab))


def decode_advance(input_ids: torch.Tensor, context_lens: torch.Tensor, positions: torch.Tensor,
                   slot_mapping: torch.Tensor, sampled: torch.Tensor, step: torch.Tensor | None = None,
                   host_ids: torch.Tensor | None = None) -> None:
    """Move a decode batch's step metadata one token forward on the device (all int64 (batch,), in place):
    input = the id sampled last step, context length + 1, position = new length - 1, slot + 1; rows whose context
    length is not positive (padding of a captured batch size) stay as they are.  ``step`` (one int64 / uint64 on the
    device): the sampler's call counter, incremented by one in the same launch.  ``host_ids`` (with ``step``): a
    pinned int64 CPU tensor (2, n >= batch + 1); row ``step & 1`` (before the increment) receives the sampled ids and
    then, in its last entry, the new counter value, written by the kernel itself: the host may read the ids as soon as
    it sees that value."""
    _C.require_cuda(input_ids, context_lens, positions, slot_mapping, sampled, step)
    n = sampled.numel()
    for t in (input_ids, context_lens, positions, slot_mapping, sampled):
        if t.dtype != torch.int64 or t.numel() < n or not t.is_contiguous():
            raise ValueError("decode_advance takes contiguous int64 tensors of at least the batch size")
    if step is not None and (step.numel() != 1 or step.element_size() != 8):
        raise ValueError("step must be one 64-bit integer on the device")
    host_ptr, host_stride = 0, 0
    if host_ids is not None:
        if step is None or host_ids.is_cuda or not host_ids.is_pinned() or host_ids.dtype != torch.int64 \
                or host_ids.dim() != 2 or host_ids.shape[0] != 2 or host_ids.shape[1] < n + 1 or not host_ids.is_contiguous():
            raise ValueError("host_ids must be a pinned contiguous int64 CPU tensor (2, >= batch + 1), given with step")
        host_ptr, host_stride = host_ids.data_ptr(), host_ids.shape[1]
    st = _C.load().mvllm_decode_advance(_ptr(input_ids), _ptr(context_lens), _ptr(positions), _ptr(slot_mapping),
                                        _ptr(sampled), _ptr(step), host_ptr, host_stride, n,
                                        _C.current_stream_ptr(sampled.device))
    _C.check(st, "decode_advance")


def _rows2d(name, t):
    if t.dim() != 2:
        raise ValueError(f"{name} must be (rows, features), got {tuple(t.shape)}")
    if t.shape[0] > 1 and t.stride(1) != 1 or t.shape[0] == 1 and t.shape[1] > 1 and t.stride(1) != 1:
        t = t.contiguous()
    return t, (t.stride(0) if t.shape[0] > 1 else t.shape[1])


def add_rms_norm(x: torch.Tensor, gamma: torch.Tensor, eps: float, residual: torch.Tensor | None = None):
    """``LayerNorm.forward`` (layers/layernorm.py:9-28) in one launch.

    Without ``residual``: returns ``x / sqrt(mean(x^2) + eps) * gamma``.  With it: returns
    ``(norm(x + residual), x + residual)``, the sum rounded to x's dtype first.  x, residual: (rows, hidden),
    rows may be strided; gamma float32 (hidden,).
    """
    _C.require_cuda(x, gamma, residual)
    x, x_stride = _rows2d("x", x)
    rows, hidden = x.shape
    if gamma.dtype != torch.float32 or gamma.numel() != hidden or not gamma.is_contiguous():
        raise ValueError(f"gamma must be contiguous float32 ({hidden},)")
    r_stride = hidden
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("residual must match x in shape and dtype")
        residual, r_stride = _rows2d("residual", residual)
    out = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    new_residual = torch.empty_like(out) if residual is not None else None
    if rows:
        lib = _C.load()
        st = lib.mvllm_add_rms_norm(_ptr(out), _ptr(new_residual), _ptr(x), _ptr(residual), _ptr(gamma), float(eps),
                                    rows, hidden, x_stride, r_stride, _C.dtype_code(x.dtype),
                                    _C.current_stream_ptr(x.device))
        _C.check(st, "add_rms_norm")
    return out if residual is None else (out, new_residual)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """``SiluAndMul.forward`` (layers/activation.py:15-18): silu(first half) * second half of the last dim."""
    _C.require_cuda(x)
    x, stride = _rows2d("x", x)
    rows, two_w = x.shape
    if two_w % 2:
        raise ValueError("the last dimension must be even")
    out = torch.empty((rows, two_w // 2), dtype=x.dtype, device=x.device)
    if rows:
        lib = _C.load()
        st = lib.mvllm_silu_and_mul(_ptr(out), _ptr(x), rows, two_w // 2, stride, _C.dtype_code(x.dtype),
                                    _C.current_stream_ptr(x.device))
        _C.check(st, "silu_and_mul")
    return out


def linear_small_m_takes(x: torch.Tensor, weight: torch.Tensor, max_rows: int = 64) -> bool:
    """Whether ``linear_small_m`` is built for this call: at most 64 rows, bf16 / fp16 on the GPU, N a multiple of 16,
    K a multiple of 512, rows of x dense."""
    return (x.is_cuda and x.dim() == 2 and 0 < x.shape[0] <= min(max_rows, 64) and x.dtype in (torch.bfloat16, torch.float16)
            and weight.dtype == x.dtype and weight.is_contiguous() and weight.shape[0] % 16 == 0
            and weight.shape[1] % 512 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0)


def linear_small_m(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` for the few rows of a decode step (the reference's projections,
    models/qwen3.py:90-94, 118, 121-160, are library GEMMs): one HIP launch in which every wave asks for its whole
    share of the weights at once, so the call costs about one memory round trip.  x (M <= 64, K), weight (N, K)
    contiguous, bias (N,) or None, all in one 16-bit dtype; fp32 accumulation.  Returns (M, N)."""
    _C.require_cuda(x, weight, bias)
    if x.dim() != 2 or weight.dim() != 2 or weight.shape[1] != x.shape[1]:
        raise ValueError(f"x (M, K) and weight (N, K) expected, got {tuple(x.shape)} and {tuple(weight.shape)}")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise ValueError("x, weight and bias must share one dtype")
    if not weight.is_contiguous() or x.stride(1) != 1:
        raise ValueError("weight must be contiguous and the rows of x dense")
    m, k = x.shape
    n = weight.shape[0]
    out = torch.empty(m, n, dtype=x.dtype, device=x.device)
    st = _C.load().mvllm_linear_small_m(_ptr(out), _ptr(x), _ptr(weight), _ptr(bias), x.stride(0) if m > 1 else k,
                                        m, n, k, _C.dtype_code(x.dtype), _C.current_stream_ptr(x.device))
    _C.check(st, "linear_small_m")
    return out


_PLAN_CACHE: dict = {}


def norm_linear_small_m_takes(x: torch.Tensor, weight: torch.Tensor, max_rows: int = 32, norm: bool = True,
                              glu: bool = False) -> bool:
    """Whether ``norm_linear_small_m`` is built for this call (``mvllm_linear_small_m_plan``, remembered per shape)."""
    if not linear_small_m_takes(x, weight, max_rows) or not x.is_contiguous():
        return False
    key = (x.shape[0], weight.shape[0], weight.shape[1], norm, glu, x.dtype)
    if key not in _PLAN_CACHE:
        st = _C.load().mvllm_linear_small_m_plan(key[0], key[1], key[2], int(norm), int(glu), _C.dtype_code(x.dtype), None)
        _PLAN_CACHE[key] = st == 0
    return _PLAN_CACHE[key]


def norm_linear_small_m(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                        gamma: torch.Tensor | None = None, eps: float = 1e-6, residual: torch.Tensor | None = None,
                        want_residual: bool = False, glu: bool = False):
    """A decode step's projection with the launches around it folded in (the reference runs them as separate
    modules, models/qwen3.py:151-160, 197-212): with ``gamma`` (float32, (K,)) the rows are first replaced by
    ``rms_norm(x + residual) * gamma`` as ``add_rms_norm`` computes it; with ``glu`` the weight is (2F, K) and the
    result ``silu(gate) * up`` as ``silu_and_mul`` computes it.  Returns the (M, N) or (M, F) product, and with
    ``want_residual`` also ``x + residual`` in x's dtype (a new tensor)."""
    _C.require_cuda(x, weight, bias, gamma, residual)
    if x.dim() != 2 or weight.dim() != 2 or weight.shape[1] != x.shape[1]:
        raise ValueError(f"x (M, K) and weight (N, K) expected, got {tuple(x.shape)} and {tuple(weight.shape)}")
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype) or (residual is not None and residual.dtype != x.dtype):
        raise ValueError("x, weight, bias and residual must share one dtype")
    if not weight.is_contiguous() or x.stride(1) != 1:
        raise ValueError("weight must be contiguous and the rows of x dense")
    m, k = x.shape
    n = weight.shape[0]
    if gamma is not None and (gamma.dtype != torch.float32 or tuple(gamma.shape) != (k,)):
        raise ValueError("gamma must be float32 of shape (K,)")
    if residual is not None and (tuple(residual.shape) != (m, k) or not residual.is_contiguous()):
        raise ValueError("residual must be a contiguous (M, K) tensor")
    if (residual is not None or want_residual) and gamma is None:
        raise ValueError("a residual needs the norm (gamma)")
    out = torch.empty(m, n // 2 if glu else n, dtype=x.dtype, device=x.device)
    res_out = torch.empty(m, k, dtype=x.dtype, device=x.device) if want_residual else None
    st = _C.load().mvllm_norm_linear_small_m(_ptr(out), _ptr(res_out), _ptr(x), _ptr(residual), _ptr(gamma), float(eps),
                                             _ptr(weight), _ptr(bias), x.stride(0) if m > 1 else k, m, n, k, int(glu),
                                             _C.dtype_code(x.dtype), _C.current_stream_ptr(x.device))
    _C.check(st, "norm_linear_small_m")
    return (out, res_out) if want_residual else out


def lm_head_sample_takes(hidden: torch.Tensor, weight: torch.Tensor, batch: int | None = None) -> bool:
    """Whether ``lm_head_sample`` is built for this call: at most 64 rows to sample, bf16 / fp16 on the GPU, a
    vocabulary that is a multiple of 16, hidden size 256, 512 or 1024."""
    rows = hidden.shape[0] if batch is None else batch
    return (hidden.is_cuda and hidden.dim() == 2 and 0 < rows <= 64 and hidden.dtype in (torch.bfloat16, torch.float16)
            and weight.dtype == hidden.dtype and weight.dim() == 2 and weight.is_contiguous()
            and weight.shape[0] % 16 == 0 and weight.shape[1] in (256, 512, 1024) and hidden.shape[1] == weight.shape[1]
            and hidden.stride(1) == 1 and hidden.stride(0) % 8 == 0 and hidden.data_ptr() % 16 == 0)


def lm_head_sample_workspace_bytes(batch: int, hidden_size: int) -> int:
    return int(_C.load().mvllm_lm_head_sample_workspace_bytes(batch, hidden_size))


def lm_head_sample(hidden: torch.Tensor, weight: torch.Tensor, temperatures: torch.Tensor, seed: int = 0,
                   offset: int = 0, row_index: torch.Tensor | None = None, out: torch.Tensor | None = None,
                   offset_dev: torch.Tensor | None = None, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """The LM head and the sampler in one pass over ``weight`` (vocab, K): the reference's
    ``ParallelLMHead.forward`` (layers/embedding_head.py:56-77) and ``SamplerLayer.forward`` (layers/sampler.py:14-19)
    without the (batch, vocab) logits.  Row ``b`` samples from ``hidden[row_index[b]]`` (``row_index`` None: row b) at
    ``temperatures[b]``; the noise is the in-kernel Philox stream of ``sample_tokens`` (same seed / offset: the same
    ids as ``sample_tokens(F.linear(hidden, weight), ...)`` up to the summation order inside a logit).  ``out``,
    ``offset_dev`` and ``workspace`` (uint8, ``lm_head_sample_workspace_bytes``) let a captured graph call it without
    allocating and draw fresh noise on every replay."""
    _C.require_cuda(hidden, weight, temperatures, row_index, out, offset_dev, workspace)
    batch = hidden.shape[0] if row_index is None else row_index.numel()
    if not lm_head_sample_takes(hidden, weight, batch):
        raise ValueError("lm_head_sample: shape or dtype not taken (see lm_head_sample_takes)")
    if temperatures.dtype != torch.float32 or temperatures.numel() != batch or not temperatures.is_contiguous():
        raise ValueError("temperatures must be contiguous float32 (batch,)")
    if row_index is not None and (row_index.dtype != torch.int64 or not row_index.is_contiguous()):
        raise ValueError("row_index must be contiguous int64")
    vocab, k = weight.shape
    if out is None:
        out = torch.empty(batch, dtype=torch.int64, device=hidden.device)
    elif out.dtype != torch.int64 or out.numel() != batch or not out.is_contiguous():
        raise ValueError("out must be contiguous int64 (batch,)")
    need = lm_head_sample_workspace_bytes(batch, k)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=hidden.device)
    st = _C.load().mvllm_lm_head_sample(_ptr(out), _ptr(hidden), hidden.stride(0) if hidden.shape[0] > 1 else k,
                                        _ptr(row_index), _ptr(weight), _ptr(temperatures), int(seed) & (2 ** 64 - 1),
                                        int(offset) & (2 ** 64 - 1), _ptr(offset_dev), batch, vocab, k,
                                        _C.dtype_code(hidden.dtype), _ptr(workspace), workspace.numel(),
                                        _C.current_stream_ptr(hidden.device))
    _C.check(st, "lm_head_sample")
    return out
