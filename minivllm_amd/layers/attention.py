"""Attention operator layer: the reference's Python surface over gfx950 HIP kernels.

Same public names, argument order, shapes and return conventions as
src/myvllm/layers/attention.py: ``store_kvcache`` (:67-108),
``flash_attention_prefill`` (:212-280), ``paged_attention_decode`` (:418-473)
and the ``Attention`` module (:476-557).  Every operator calls
libminivllm_amd.so through ctypes on the current torch stream; there is no
Triton, no PyTorch fallback and no CPU path.

Additions with no counterpart in the reference: the INT8 KV-cache operators
``store_kvcache_int8`` / ``paged_attention_decode_int8`` and the
``kv_cache_dtype="int8"`` mode of ``Attention``.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from minivllm_amd import _C
from minivllm_amd.layers.fused import qk_norm_rope_store
from minivllm_amd.utils.context import get_context

__all__ = [
    "store_kvcache", "store_kvcache_int8", "flash_attention_prefill", "flash_attention_prefill_paged",
    "flash_attention_prefill_paged_int8",
    "paged_attention_decode", "paged_attention_decode_int8", "decode_workspace_bytes", "paged_decode_plan",
    "prefill_plan", "Attention",
]

_workspaces: dict = {}   # device index -> uint8 tensor reused by decode calls on that device that bring no workspace
_retired: list = []      # outgrown workspaces: kept alive, because a captured hipGraph may hold their address


def _decode_workspace(device: torch.device, nbytes: int, own: torch.Tensor | None = None):
    """Split-K scratch for paged decode.  ``own`` (a caller-owned uint8 tensor, e.g. the model runner's, sized
    before its graphs were captured) is used when it is large enough; otherwise one buffer per device, grown on
    demand and never freed: a buffer that has been handed out may be referenced by a captured graph."""
    if nbytes == 0:
        return None
    if own is not None and own.numel() >= nbytes:
        return own
    key = device.index if device.index is not None else torch.cuda.current_device()
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def decode_workspace_bytes(batch: int, num_heads: int, head_dim: int, max_num_blocks: int, block_size: int) -> int:
    """Bytes of split-K scratch a decode call of these static sizes may use (host arithmetic only)."""
    return int(_C.load().mvllm_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_num_blocks, block_size))


def _ptr(t):
    return 0 if t is None else t.data_ptr()


_shapes_seen: set = set()    # (operation, heads, kv heads, head_dim, block_size, dtype, int8) already checked


def _warn_if_generic(op: str, num_heads: int, num_kv_heads: int, head_dim: int, block_size: int, dtype, int8: bool):
    """One warning per shape when a call runs on a generic kernel (a correctness path, about two orders of magnitude
    slower than the MFMA kernels).  The reference's Triton kernels tile any power-of-two head_dim
    (attention.py:249-257, 453); here the fast kernels cover head_dim 128 and 64 (bf16 / fp16 also 32, 80, 96, 112 and 256),
    blocks of a multiple of 16 tokens (decode at head_dim 128 / 64 also 1, 2, 4 and 8; prefill any size when the
    caller passes max_seqlen_k) and any number of query heads per kv head (decode streams a kv head once per 16 of
    them)."""
    key = (op, num_heads, num_kv_heads, head_dim, block_size, dtype, int8)
    if key in _shapes_seen:
        return
    _shapes_seen.add(key)
    if op == "decode":
        generic = paged_decode_plan(1, num_heads, num_kv_heads, head_dim, 1, block_size, dtype, int8)[2] == 0
    else:
        generic = prefill_plan(num_heads, num_kv_heads, head_dim, block_size, dtype, int8) == 0
    if generic:
        import warnings
        warnings.warn(f"minivllm_amd {op}: no MFMA kernel for num_heads={num_heads}, num_kv_heads={num_kv_heads}, "
                      f"head_dim={head_dim}, block_size={block_size}, {dtype}{', int8 cache' if int8 else ''}; "
                      "running on the generic kernel (correct, but roughly 100x slower)", RuntimeWarning, stacklevel=3)


def _check_cache(name, cache, num_kv_heads, head_dim):
    if cache.dim() != 4 or cache.shape[2] != num_kv_heads or cache.shape[3] != head_dim:
        raise ValueError(f"{name} must be [num_blocks, block_size, {num_kv_heads}, {head_dim}], got "
                         f"{tuple(cache.shape)}")
    if not cache.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _slots(slot_mapping):
    if slot_mapping.dtype != torch.int64:
        slot_mapping = slot_mapping.to(torch.int64)
    return slot_mapping.contiguous()


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor, block_size: int) -> None:
    """Scatter K/V token rows into the paged caches (in place).

    key/value: (num_tokens, num_kv_heads, head_dim); k/v_cache:
    (num_blocks, block_size, num_kv_heads, head_dim); slot_mapping:
    (num_tokens,) flat slot per token, -1 = skip.  Reference: attention.py:67-108.
    """
    num_tokens, num_kv_heads, head_dim = key.shape
    assert k_cache.shape == v_cache.shape, "K and V cache shapes must match"
    assert slot_mapping.numel() == num_tokens, "Slot mapping size must match number of tokens"
    _C.require_cuda(key, value, k_cache, v_cache, slot_mapping)
    if value.shape != key.shape:
        raise ValueError("key and value shapes must match")
    if key.dtype != k_cache.dtype or value.dtype != v_cache.dtype:
        raise ValueError(f"store_kvcache is a same-dtype copy: key {key.dtype}, cache {k_cache.dtype}")
    _check_cache("k_cache", k_cache, num_kv_heads, head_dim)
    _check_cache("v_cache", v_cache, num_kv_heads, head_dim)
    key = key.contiguous()
    value = value.contiguous()
    slots = _slots(slot_mapping)
    num_slots = k_cache.shape[0] * k_cache.shape[1]
    lib = _C.load()
    st = lib.mvllm_store_kvcache(_ptr(key), _ptr(value), _ptr(k_cache), _ptr(v_cache), _ptr(slots),
                                 num_tokens, num_slots, num_kv_heads, head_dim,
                                 _C.dtype_code(key.dtype), _C.current_stream_ptr(key.device))
    _C.check(st, "store_kvcache")


def store_kvcache_int8(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       k_scale: torch.Tensor, v_scale: torch.Tensor, slot_mapping: torch.Tensor,
                       block_size: int) -> None:
    """Quantise each (token, kv head) vector to int8 (scale = absmax/127) and scatter.

    k/v_cache: int8 (num_blocks, block_size, Hkv, D); k/v_scale: float32
    (num_blocks, block_size, Hkv).  Otherwise as ``store_kvcache``.
    """
    num_tokens, num_kv_heads, head_dim = key.shape
    assert k_cache.shape == v_cache.shape, "K and V cache shapes must match"
    assert slot_mapping.numel() == num_tokens, "Slot mapping size must match number of tokens"
    _C.require_cuda(key, value, k_cache, v_cache, k_scale, v_scale, slot_mapping)
    if value.shape != key.shape or value.dtype != key.dtype:
        raise ValueError("key and value must have the same shape and dtype")
    if k_cache.dtype != torch.int8 or v_cache.dtype != torch.int8:
        raise ValueError("int8 caches expected")
    _check_cache("k_cache", k_cache, num_kv_heads, head_dim)
    _check_cache("v_cache", v_cache, num_kv_heads, head_dim)
    for name, s in (("k_scale", k_scale), ("v_scale", v_scale)):
        if s.dtype != torch.float32 or tuple(s.shape) != tuple(k_cache.shape[:3]) or not s.is_contiguous():
            raise ValueError(f"{name} must be contiguous float32 {tuple(k_cache.shape[:3])}")
    key = key.contiguous()
    value = value.contiguous()
    slots = _slots(slot_mapping)
    num_slots = k_cache.shape[0] * k_cache.shape[1]
    lib = _C.load()
    st = lib.mvllm_store_kvcache_int8(_ptr(key), _ptr(value), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale),
                                      _ptr(v_scale), _ptr(slots), num_tokens, num_slots, num_kv_heads,
                                      head_dim, _C.dtype_code(key.dtype), _C.current_stream_ptr(key.device))
    _C.check(st, "store_kvcache_int8")


def flash_attention_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor,
                            scale: float, num_heads: int, num_kv_heads: int, head_dim: int) -> torch.Tensor:
    """Causal attention over a packed ragged batch.  Reference: attention.py:212-280.

    q: (total_tokens, num_heads, head_dim); k, v: (total_tokens, num_kv_heads,
    head_dim); cu_seqlens: int32 (num_seqs + 1,).  Returns a tensor like q.
    No device->host synchronisation happens here.
    """
    _C.require_cuda(q, k, v, cu_seqlens)
    if q.dim() != 3 or tuple(q.shape[1:]) != (num_heads, head_dim):
        raise ValueError(f"q must be (total_tokens, {num_heads}, {head_dim}), got {tuple(q.shape)}")
    total = q.shape[0]
    for name, t in (("k", k), ("v", v)):
        if tuple(t.shape) != (total, num_kv_heads, head_dim):
            raise ValueError(f"{name} must be ({total}, {num_kv_heads}, {head_dim}), got {tuple(t.shape)}")
        if t.dtype != q.dtype:
            raise ValueError("q, k and v must share one dtype")
    q = q.contiguous()
    k = k.contiguous()
    v = v.contiguous()
    if cu_seqlens.dtype != torch.int32:
        cu_seqlens = cu_seqlens.to(torch.int32)
    cu_seqlens = cu_seqlens.contiguous()
    output = torch.empty_like(q)
    num_seqs = cu_seqlens.shape[0] - 1
    _warn_if_generic("prefill", num_heads, num_kv_heads, head_dim, 0, q.dtype, False)
    lib = _C.load()
    st = lib.mvllm_prefill_varlen(_ptr(output), _ptr(q), _ptr(k), _ptr(v), _ptr(cu_seqlens), num_seqs, total,
                                  num_heads, num_kv_heads, head_dim, float(scale), _C.dtype_code(q.dtype),
                                  _C.current_stream_ptr(q.device))
    _C.check(st, "flash_attention_prefill")
    return output


def flash_attention_prefill_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                  block_tables: torch.Tensor, cu_seqlens_q: torch.Tensor,
                                  cu_seqlens_k: torch.Tensor, scale: float, num_heads: int, num_kv_heads: int,
                                  head_dim: int, block_size: int, max_seqlen_k: int | None = None,
                                  key_splits: int | None = None) -> torch.Tensor:
    """Causal prefill of the tokens that follow each sequence's cached prefix, with every key read from the
    paged cache.  Consumes the metadata ``ModelRunner.prepare_prefill`` builds for prefix-cache hits
    (model_runner.py:192-226), which the reference's ``Attention.forward`` ignores (attention.py:518-523).

    q: (total_new_tokens, num_heads, head_dim) packed by ``cu_seqlens_q``; caches
    (num_blocks, block_size, Hkv, D) already holding all ``cu_seqlens_k`` keys of every sequence;
    block_tables int32 (num_seqs, max_num_blocks).  Returns a tensor like q.
    A block size that is not a multiple of 16 (8, 1, 24 ...) runs on the generic kernel unless ``max_seqlen_k`` (the
    host's upper bound of every sequence's key count, ``Context.max_seqlen_k``) is given: the batch's keys and values
    are then copied into a temporary cache of 16-token blocks (``STAGED_PREFILL_MAX_BYTES`` at most) and the MFMA
    kernels run over that.
    With ``max_seqlen_k`` given, a batch of few new tokens behind long prefixes (too few query tiles to occupy the
    chip) has every sequence's keys cut into ranges that are walked side by side and merged; ``key_splits`` forces the
    number of ranges (0 or 1: never split; None: the library's ``mvllm_prefill_paged_split_plan`` decides).
    """
    _C.require_cuda(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k)
    if q.dim() != 3 or tuple(q.shape[1:]) != (num_heads, head_dim):
        raise ValueError(f"q must be (total_tokens, {num_heads}, {head_dim}), got {tuple(q.shape)}")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise ValueError(f"q {q.dtype} and cache {k_cache.dtype} dtypes differ (for an int8 cache use flash_attention_prefill_paged_int8)")
    _check_cache("k_cache", k_cache, num_kv_heads, head_dim)
    _check_cache("v_cache", v_cache, num_kv_heads, head_dim)
    if k_cache.shape != v_cache.shape:
        raise ValueError("K and V cache shapes must match")
    if k_cache.shape[1] != block_size:
        raise ValueError(f"cache block dimension {k_cache.shape[1]} != block_size {block_size}")
    num_seqs = cu_seqlens_q.shape[0] - 1
    if cu_seqlens_k.shape[0] != num_seqs + 1:
        raise ValueError("cu_seqlens_q and cu_seqlens_k must have the same length")
    if block_tables.dim() != 2 or block_tables.shape[0] != num_seqs:
        raise ValueError(f"block_tables must be ({num_seqs}, max_num_blocks), got {tuple(block_tables.shape)}")
    q = q.contiguous()
    block_tables = block_tables.to(torch.int32).contiguous()
    cu_seqlens_q = cu_seqlens_q.to(torch.int32).contiguous()
    cu_seqlens_k = cu_seqlens_k.to(torch.int32).contiguous()
    output = torch.empty_like(q)
    lib = _C.load()
    if max_seqlen_k is not None and int(max_seqlen_k) > 0 and block_size % 16 != 0:
        need = lib.mvllm_prefill_paged_staged_workspace_bytes(num_seqs, int(max_seqlen_k), num_heads, num_kv_heads, head_dim,
                                                              _C.dtype_code(q.dtype), 0)
        if 0 < need <= STAGED_PREFILL_MAX_BYTES:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            st = lib.mvllm_prefill_paged_staged(_ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                                block_tables.shape[1], _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs,
                                                q.shape[0], int(max_seqlen_k), num_heads, num_kv_heads, head_dim, block_size,
                                                k_cache.shape[0], float(scale), _C.dtype_code(q.dtype), _ptr(workspace), need,
                                                _C.current_stream_ptr(q.device))
            _C.check(st, "flash_attention_prefill_paged (staged)")
            return output
    if max_seqlen_k is not None and int(max_seqlen_k) > 0 and q.dtype != torch.float32:
        code = _C.dtype_code(q.dtype)
        splits = key_splits
        if splits is None:
            splits = lib.mvllm_prefill_paged_split_plan(num_seqs, q.shape[0], int(max_seqlen_k), num_heads, num_kv_heads,
                                                        head_dim, block_size, code, 0)
        need = 0
        if splits >= 2:
            need = lib.mvllm_prefill_paged_split_workspace_bytes(num_seqs, q.shape[0], int(max_seqlen_k), num_heads,
                                                                 num_kv_heads, head_dim, block_size, code, splits)
            if key_splits is not None and need == 0:
                raise ValueError(f"key_splits={key_splits}: the split form is not built for this shape")
        if 0 < need <= STAGED_PREFILL_MAX_BYTES:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            st = lib.mvllm_prefill_paged_split(_ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                               block_tables.shape[1], _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs,
                                               q.shape[0], int(max_seqlen_k), num_heads, num_kv_heads, head_dim, block_size,
                                               k_cache.shape[0], float(scale), code, splits, _ptr(workspace), need,
                                               _C.current_stream_ptr(q.device))
            _C.check(st, "flash_attention_prefill_paged (split over keys)")
            return output
    _warn_if_generic("prefill", num_heads, num_kv_heads, head_dim, block_size, q.dtype, False)
    st = lib.mvllm_prefill_paged(_ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                 block_tables.shape[1], _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs,
                                 q.shape[0], num_heads, num_kv_heads, head_dim, block_size, k_cache.shape[0],
                                 float(scale), _C.dtype_code(q.dtype), _C.current_stream_ptr(q.device))
    _C.check(st, "flash_attention_prefill_paged")
    return output


STAGED_PREFILL_MAX_BYTES = 4 << 30    # larger temporary caches are not asked for: the call then runs in one step


def flash_attention_prefill_paged_int8(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                       k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor,
                                       cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor, scale: float,
                                       num_heads: int, num_kv_heads: int, head_dim: int, block_size: int,
                                       max_seqlen_k: int | None = None, key_splits: int | None = None) -> torch.Tensor:
    """``flash_attention_prefill_paged`` over an INT8 cache written by ``store_kvcache_int8``: every key, the new
    tokens' included, is read from the cache and dequantised in the kernel, as decode does for the same tokens.
    q bf16 / fp16; caches int8 (num_blocks, block_size, Hkv, D); scales float32 (num_blocks, block_size, Hkv).
    ``max_seqlen_k`` (the host's upper bound of every sequence's key count, ``Context.max_seqlen_k``) lets the call
    run in two steps: the batch's keys and values are dequantised once into a temporary 16-bit cache
    (2 x num_seqs x max_seqlen_k x Hkv x D x 2 bytes from torch's allocator, at most ``STAGED_PREFILL_MAX_BYTES``),
    which is a quarter faster than converting every tile for every query tile that walks it, and the only MFMA path
    for block sizes that are not a multiple of 16.  Few new tokens behind long prefixes are instead cut over the keys
    as in ``flash_attention_prefill_paged`` (``key_splits`` as there)."""
    _C.require_cuda(q, k_cache, v_cache, k_scale, v_scale, block_tables, cu_seqlens_q, cu_seqlens_k)
    if q.dim() != 3 or tuple(q.shape[1:]) != (num_heads, head_dim):
        raise ValueError(f"q must be (total_tokens, {num_heads}, {head_dim}), got {tuple(q.shape)}")
    if k_cache.dtype != torch.int8 or v_cache.dtype != torch.int8:
        raise ValueError("int8 caches expected")
    _check_cache("k_cache", k_cache, num_kv_heads, head_dim)
    _check_cache("v_cache", v_cache, num_kv_heads, head_dim)
    if k_cache.shape != v_cache.shape or k_cache.shape[1] != block_size:
        raise ValueError("K and V cache shapes must match and have block_size rows per block")
    for name, sc in (("k_scale", k_scale), ("v_scale", v_scale)):
        if sc.dtype != torch.float32 or tuple(sc.shape) != tuple(k_cache.shape[:3]) or not sc.is_contiguous():
            raise ValueError(f"{name} must be contiguous float32 {tuple(k_cache.shape[:3])}")
    num_seqs = cu_seqlens_q.shape[0] - 1
    if cu_seqlens_k.shape[0] != num_seqs + 1:
        raise ValueError("cu_seqlens_q and cu_seqlens_k must have the same length")
    if block_tables.dim() != 2 or block_tables.shape[0] != num_seqs:
        raise ValueError(f"block_tables must be ({num_seqs}, max_num_blocks), got {tuple(block_tables.shape)}")
    q = q.contiguous()
    block_tables = block_tables.to(torch.int32).contiguous()
    cu_seqlens_q = cu_seqlens_q.to(torch.int32).contiguous()
    cu_seqlens_k = cu_seqlens_k.to(torch.int32).contiguous()
    output = torch.empty_like(q)
    if max_seqlen_k is not None and int(max_seqlen_k) > 0:
        lib, code = _C.load(), _C.dtype_code(q.dtype)
        splits = key_splits
        if splits is None:
            splits = lib.mvllm_prefill_paged_split_plan(num_seqs, q.shape[0], int(max_seqlen_k), num_heads, num_kv_heads,
                                                        head_dim, block_size, code, 1)
        need = 0
        if splits >= 2:
            need = lib.mvllm_prefill_paged_split_workspace_bytes(num_seqs, q.shape[0], int(max_seqlen_k), num_heads,
                                                                 num_kv_heads, head_dim, block_size, code, splits)
            if key_splits is not None and need == 0:
                raise ValueError(f"key_splits={key_splits}: the split form is not built for this shape")
        if 0 < need <= STAGED_PREFILL_MAX_BYTES:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            st = lib.mvllm_prefill_paged_int8_split(
                _ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale), _ptr(block_tables),
                block_tables.shape[1], _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs, q.shape[0], int(max_seqlen_k),
                num_heads, num_kv_heads, head_dim, block_size, k_cache.shape[0], float(scale), code, splits,
                _ptr(workspace), need, _C.current_stream_ptr(q.device))
            _C.check(st, "flash_attention_prefill_paged_int8 (split over keys)")
            return output
        need = _C.load().mvllm_prefill_paged_staged_workspace_bytes(num_seqs, int(max_seqlen_k), num_heads, num_kv_heads,
                                                                    head_dim, _C.dtype_code(q.dtype), 1)
        if 0 < need <= STAGED_PREFILL_MAX_BYTES:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            st = _C.load().mvllm_prefill_paged_int8_staged(
                _ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale), _ptr(v_scale), _ptr(block_tables),
                block_tables.shape[1], _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs, q.shape[0], int(max_seqlen_k),
                num_heads, num_kv_heads, head_dim, block_size, k_cache.shape[0], float(scale), _C.dtype_code(q.dtype),
                _ptr(workspace), need, _C.current_stream_ptr(q.device))
            _C.check(st, "flash_attention_prefill_paged_int8 (staged)")
            return output
    st = _C.load().mvllm_prefill_paged_int8(_ptr(output), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale),
                                            _ptr(v_scale), _ptr(block_tables), block_tables.shape[1],
                                            _ptr(cu_seqlens_q), _ptr(cu_seqlens_k), num_seqs, q.shape[0], num_heads,
                                            num_kv_heads, head_dim, block_size, k_cache.shape[0], float(scale),
                                            _C.dtype_code(q.dtype), _C.current_stream_ptr(q.device))
    _C.check(st, "flash_attention_prefill_paged_int8")
    return output


def _decode_common(query, k_cache, v_cache, block_tables, context_lens, num_heads, num_kv_heads, head_dim,
                   block_size):
    if query.dim() != 3 or tuple(query.shape[1:]) != (num_heads, head_dim):
        raise ValueError(f"query must be (batch, {num_heads}, {head_dim}), got {tuple(query.shape)}")
    _check_cache("k_cache", k_cache, num_kv_heads, head_dim)
    _check_cache("v_cache", v_cache, num_kv_heads, head_dim)
    if k_cache.shape != v_cache.shape:
        raise ValueError("K and V cache shapes must match")
    if k_cache.shape[1] != block_size:
        raise ValueError(f"cache block dimension {k_cache.shape[1]} != block_size {block_size}")
    batch = query.shape[0]
    if block_tables is None or context_lens is None:
        raise ValueError("block_tables and context_lens must be provided for paged decode")
    if block_tables.dim() != 2 or block_tables.shape[0] != batch:
        raise ValueError(f"block_tables must be ({batch}, max_num_blocks), got {tuple(block_tables.shape)}")
    if context_lens.numel() != batch:
        raise ValueError("context_lens must have one entry per sequence")
    if block_tables.dtype != torch.int32:
        block_tables = block_tables.to(torch.int32)
    block_tables = block_tables.contiguous()
    if context_lens.dtype not in (torch.int32, torch.int64):
        context_lens = context_lens.to(torch.int64)
    context_lens = context_lens.contiguous()
    return query.contiguous(), block_tables, context_lens


def paged_decode_plan(batch: int, num_heads: int, num_kv_heads: int, head_dim: int, max_num_blocks: int,
                      block_size: int, dtype: torch.dtype = torch.bfloat16, int8_cache: bool = False):
    """(part_tokens, num_parts, waves_per_head) a decode call of these static sizes runs with (host arithmetic only).
    waves_per_head: 1 = one wave per kv head walks a partition, >1 = the small-batch form (that many waves share
    one kv head's partition), 0 = the generic kernel."""
    import ctypes
    out = [ctypes.c_int(0) for _ in range(3)]
    st = _C.load().mvllm_paged_decode_plan(batch, num_heads, num_kv_heads, head_dim, max_num_blocks, block_size,
                                           _C.dtype_code(dtype), int(int8_cache), *[ctypes.byref(x) for x in out])
    _C.check(st, "paged_decode_plan")
    return tuple(x.value for x in out)


def prefill_plan(num_heads: int, num_kv_heads: int, head_dim: int, block_size: int = 0,
                 dtype: torch.dtype = torch.bfloat16, int8_cache: bool = False) -> int:
    """Kernel a prefill of these static sizes runs on (host arithmetic only): 2 = LDS-tiled MFMA kernel, 1 = 16-row
    tile MFMA kernel, 0 = generic kernel, -1 = unsupported.  block_size 0 = packed prefill, > 0 = over a paged cache."""
    import ctypes
    out = ctypes.c_int(0)
    st = _C.load().mvllm_prefill_plan(num_heads, num_kv_heads, head_dim, block_size, _C.dtype_code(dtype),
                                      int(int8_cache), ctypes.byref(out))
    _C.check(st, "prefill_plan")
    return out.value


def paged_attention_decode(query: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_tables: torch.Tensor, context_lens: torch.Tensor, scale: float,
                           num_heads: int, num_kv_heads: int, head_dim: int, block_size: int, *,
                           workspace: torch.Tensor | None = None) -> torch.Tensor:
    """One query token per sequence over its paged KV.  Reference: attention.py:418-473.

    query: (batch, num_heads, head_dim); caches (num_blocks, block_size, Hkv, D);
    block_tables int32 (batch, max_num_blocks), -1 padded; context_lens int32 or
    int64 (batch,).  Returns a tensor like query; rows with context_len 0 are zeros.
    ``workspace`` (optional, not in the reference): a uint8 device tensor the caller owns for the split-K
    partials; without it, or when it is too small, a per-device buffer of this module is used.
    """
    _C.require_cuda(query, k_cache, v_cache, block_tables, context_lens)
    if k_cache.dtype != query.dtype or v_cache.dtype != query.dtype:
        raise ValueError(f"query {query.dtype} and cache {k_cache.dtype} dtypes differ")
    query, block_tables, context_lens = _decode_common(query, k_cache, v_cache, block_tables, context_lens,
                                                       num_heads, num_kv_heads, head_dim, block_size)
    batch, max_blocks = block_tables.shape
    output = torch.empty_like(query)
    if batch == 0:
        return output
    _warn_if_generic("decode", num_heads, num_kv_heads, head_dim, block_size, query.dtype, False)
    lib = _C.load()
    nbytes = lib.mvllm_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks, block_size)
    ws = _decode_workspace(query.device, nbytes, workspace)
    st = lib.mvllm_paged_decode(_ptr(output), _ptr(query), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                                max_blocks, _ptr(context_lens), int(context_lens.dtype == torch.int64), batch,
                                num_heads, num_kv_heads, head_dim, block_size, k_cache.shape[0], float(scale),
                                _C.dtype_code(query.dtype), _ptr(ws), 0 if ws is None else ws.numel(),
                                _C.current_stream_ptr(query.device))
    _C.check(st, "paged_attention_decode")
    return output


def paged_attention_decode_int8(query: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                k_scale: torch.Tensor, v_scale: torch.Tensor, block_tables: torch.Tensor,
                                context_lens: torch.Tensor, scale: float, num_heads: int, num_kv_heads: int,
                                head_dim: int, block_size: int, *,
                                workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Paged decode over an int8 cache written by ``store_kvcache_int8`` (``workspace`` as in
    ``paged_attention_decode``)."""
    _C.require_cuda(query, k_cache, v_cache, k_scale, v_scale, block_tables, context_lens)
    if k_cache.dtype != torch.int8 or v_cache.dtype != torch.int8:
        raise ValueError("int8 caches expected")
    query, block_tables, context_lens = _decode_common(query, k_cache, v_cache, block_tables, context_lens,
                                                       num_heads, num_kv_heads, head_dim, block_size)
    for name, s in (("k_scale", k_scale), ("v_scale", v_scale)):
        if s.dtype != torch.float32 or tuple(s.shape) != tuple(k_cache.shape[:3]) or not s.is_contiguous():
            raise ValueError(f"{name} must be contiguous float32 {tuple(k_cache.shape[:3])}")
    batch, max_blocks = block_tables.shape
    output = torch.empty_like(query)
    if batch == 0:
        return output
    _warn_if_generic("decode", num_heads, num_kv_heads, head_dim, block_size, query.dtype, True)
    lib = _C.load()
    nbytes = lib.mvllm_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks, block_size)
    ws = _decode_workspace(query.device, nbytes, workspace)
    st = lib.mvllm_paged_decode_int8(_ptr(output), _ptr(query), _ptr(k_cache), _ptr(v_cache), _ptr(k_scale),
                                     _ptr(v_scale), _ptr(block_tables), max_blocks, _ptr(context_lens),
                                     int(context_lens.dtype == torch.int64), batch, num_heads, num_kv_heads,
                                     head_dim, block_size, k_cache.shape[0], float(scale),
                                     _C.dtype_code(query.dtype), _ptr(ws), 0 if ws is None else ws.numel(),
                                     _C.current_stream_ptr(query.device))
    _C.check(st, "paged_attention_decode_int8")
    return output


class Attention(nn.Module):
    """Dispatches on the engine ``Context``: optional KV store, then varlen
    prefill or paged decode.  Reference: attention.py:476-557.

    ``k_cache`` / ``v_cache`` are assigned from outside (views of the engine's
    pool, ``[num_blocks, block_size, Hkv, D]``); until then they are empty and
    the store is skipped.  With ``kv_cache_dtype="int8"`` the caches are int8
    and ``k_scale`` / ``v_scale`` (float32 ``[num_blocks, block_size, Hkv]``)
    must be assigned too.
    """

    def __init__(self, num_heads: int, head_dim: int, scale: float = 1.0, num_kv_heads: int = None,
                 block_size: int = 16, kv_cache_dtype: str = "auto"):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads if num_kv_heads is not None else num_heads
        self.block_size = block_size
        if kv_cache_dtype not in ("auto", "int8"):
            raise ValueError("kv_cache_dtype must be 'auto' or 'int8'")
        self.kv_cache_dtype = kv_cache_dtype
        self.k_cache = self.v_cache = torch.tensor([])
        self.k_scale = self.v_scale = torch.tensor([])
        self.decode_workspace = None      # optional split-K scratch assigned from outside, like the caches

    def forward_fused(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
                      cos_sin_cache: torch.Tensor, gamma: torch.Tensor | None, eps: float) -> torch.Tensor:
        """``forward`` on q, k, v as they leave the QKV projection: the caller's RMSNorm of q and k (one
        float32 ``gamma`` over head_dim, None = no norm), the rotary embedding at ``positions`` and the cache
        store run in one launch in front of the prefill or decode kernel (qwen3.py:104-110)."""
        context = get_context()
        int8 = self.kv_cache_dtype == "int8"
        store = self.k_cache.numel() > 0 and self.v_cache.numel() > 0 and context.slot_mapping is not None
        if q.dim() == 4:          # (B, N, H, D) -> (B*N, H, D)
            q, k, v = (t.reshape(-1, t.shape[-2], t.shape[-1]) for t in (q, k, v))
        q, k, v = qk_norm_rope_store(
            q, k, v, positions, cos_sin_cache, gamma, eps,
            slot_mapping=context.slot_mapping if store else None,
            k_cache=self.k_cache if store else None, v_cache=self.v_cache if store else None,
            k_scale=self.k_scale if store and int8 else None, v_scale=self.v_scale if store and int8 else None,
            need_kv=context.is_prefill and context.block_tables is None)
        return self._attend(context, q, k, v)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        context = get_context()
        k_cache, v_cache = self.k_cache, self.v_cache
        int8 = self.kv_cache_dtype == "int8"

        if k_cache.numel() > 0 and v_cache.numel() > 0 and context.slot_mapping is not None:
            if k.dim() == 4:      # (B, N, Hkv, D) -> (B*N, Hkv, D)
                k_rows = k.reshape(-1, k.shape[-2], k.shape[-1])
                v_rows = v.reshape(-1, v.shape[-2], v.shape[-1])
            else:
                k_rows, v_rows = k, v
            if int8:
                store_kvcache_int8(k_rows, v_rows, k_cache, v_cache, self.k_scale, self.v_scale,
                                   context.slot_mapping, self.block_size)
            else:
                store_kvcache(k_rows, v_rows, k_cache, v_cache, context.slot_mapping, self.block_size)

        return self._attend(context, q, k, v)

    def _attend(self, context, q, k, v):
        k_cache, v_cache = self.k_cache, self.v_cache
        int8 = self.kv_cache_dtype == "int8"
        scale = self.scale / (self.head_dim ** 0.5)

        if context.is_prefill:
            if q.dim() == 4:
                # Batched mode (B, N, Hq, D): B sequences of N tokens each.  The reference dispatches to a function
                # it never defines (attention.py:526-533); here the batch is the packed case with equal lengths.
                bsz, n = q.shape[:2]
                cu = torch.arange(bsz + 1, dtype=torch.int32, device=q.device) * n
                if context.block_tables is not None:
                    # ... over cached prefixes: every sequence brings N new tokens, its keys (prefix + new) are
                    # counted by cu_seqlens_k and read from the paged cache, which the store above has completed
                    if context.cu_seqlens_k is None or k_cache.numel() == 0:
                        raise ValueError("cu_seqlens_k and the KV cache must be provided for prefill over a cached prefix")
                    q_rows = q.reshape(bsz * n, self.num_heads, self.head_dim)
                    if int8:
                        o = flash_attention_prefill_paged_int8(q_rows, k_cache, v_cache, self.k_scale, self.v_scale,
                                                               context.block_tables, cu, context.cu_seqlens_k, scale,
                                                               self.num_heads, self.num_kv_heads, self.head_dim,
                                                               self.block_size, context.max_seqlen_k or None)
                    else:
                        o = flash_attention_prefill_paged(q_rows, k_cache, v_cache, context.block_tables, cu,
                                                          context.cu_seqlens_k, scale, self.num_heads,
                                                          self.num_kv_heads, self.head_dim, self.block_size,
                                                          context.max_seqlen_k or None)
                    return o.reshape(bsz, n, self.num_heads * self.head_dim)
                o = flash_attention_prefill(q.reshape(bsz * n, self.num_heads, self.head_dim),
                                            k.reshape(bsz * n, self.num_kv_heads, self.head_dim),
                                            v.reshape(bsz * n, self.num_kv_heads, self.head_dim), cu, scale,
                                            self.num_heads, self.num_kv_heads, self.head_dim)
                return o.reshape(bsz, n, self.num_heads * self.head_dim)
            if q.dim() != 3:
                raise ValueError("prefill expects q of shape (total_tokens, num_heads, head_dim) or "
                                 "(batch, tokens, num_heads, head_dim)")
            cu_seqlens = context.cu_seqlens_q
            if cu_seqlens is None:
                raise ValueError("cu_seqlens_q must be provided for varlen attention")
            if context.block_tables is not None:
                # some sequence starts after a cached prefix: every key comes from the paged cache, which the
                # store above has just completed with the new tokens (model_runner.py:206-215)
                if context.cu_seqlens_k is None or k_cache.numel() == 0:
                    raise ValueError("cu_seqlens_k and the KV cache must be provided for prefill over a cached prefix")
                if int8:
                    o = flash_attention_prefill_paged_int8(q, k_cache, v_cache, self.k_scale, self.v_scale,
                                                           context.block_tables, cu_seqlens, context.cu_seqlens_k,
                                                           scale, self.num_heads, self.num_kv_heads, self.head_dim,
                                                           self.block_size, context.max_seqlen_k or None)
                else:
                    o = flash_attention_prefill_paged(q, k_cache, v_cache, context.block_tables, cu_seqlens,
                                                      context.cu_seqlens_k, scale, self.num_heads, self.num_kv_heads,
                                                      self.head_dim, self.block_size, context.max_seqlen_k or None)
                return o.reshape(o.shape[0], self.num_heads * self.head_dim)
            o = flash_attention_prefill(q, k, v, cu_seqlens, scale, self.num_heads, self.num_kv_heads,
                                        self.head_dim)
            return o.reshape(o.shape[0], self.num_heads * self.head_dim)

        if q.dim() == 4:          # (B, 1, Hq, D) -> (B, Hq, D)
            q = q.squeeze(1)
        if int8:
            o = paged_attention_decode_int8(q, k_cache, v_cache, self.k_scale, self.v_scale,
                                            context.block_tables, context.context_lens, scale,
                                            self.num_heads, self.num_kv_heads, self.head_dim, self.block_size,
                                            workspace=self.decode_workspace)
        else:
            o = paged_attention_decode(q, k_cache, v_cache, context.block_tables, context.context_lens, scale,
                                       self.num_heads, self.num_kv_heads, self.head_dim, self.block_size,
                                       workspace=self.decode_workspace)
        return o.reshape(o.shape[0], self.num_heads * self.head_dim)
