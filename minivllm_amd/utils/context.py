"""Per-step engine -> kernel metadata record.

Mirrors src/myvllm/utils/context.py:5-27 field for field (order matters:
``set_context`` is positional-compatible).  The record is replaced, never
mutated, by ``set_context`` / ``reset_context``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class Context:
    is_prefill: bool = False
    cu_seqlens_q: Optional[torch.Tensor] = None     # int32 [B+1]
    cu_seqlens_k: Optional[torch.Tensor] = None     # int32 [B+1]
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    slot_mapping: Optional[torch.Tensor] = None     # int64 [T], -1 = do not store
    context_lens: Optional[torch.Tensor] = None     # int64 (engine) or int32 [B]
    block_tables: Optional[torch.Tensor] = None     # int32 [B, MB], -1 padded


_context = Context()


def get_context() -> Context:
    return _context


def reset_context() -> None:
    global _context
    _context = Context()


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0,
                slot_mapping=None, context_lens=None, block_tables=None) -> None:
    global _context
    _context = Context(is_prefill, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                       slot_mapping, context_lens, block_tables)
