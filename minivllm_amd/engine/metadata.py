"""Per-step metadata producers: plain-integer versions of
``ModelRunner.prepare_prefill`` / ``prepare_decode`` (src/myvllm/engine/model_runner.py:180-256).

They return Python lists; ``ModelRunner`` turns them into pinned tensors and
the ``Context``.  ``reuse_cached_kv`` selects whether tokens covered by
prefix-cache hits are skipped (the reference's layout, which needs a prefill
kernel that reads the paged cache) or recomputed (what the engine does today:
shared blocks are rewritten with identical values).
"""
from __future__ import annotations


def prefill_metadata(seqs, block_size: int, reuse_cached_kv: bool = True) -> dict:
    input_ids, slot_mapping = [], []
    cu_q, cu_k = [0], [0]
    max_q = max_k = 0
    for seq in seqs:
        cached = seq.num_cached_tokens if reuse_cached_kv else 0
        n = len(seq)
        input_ids.extend(seq.token_ids[cached:])
        cu_q.append(cu_q[-1] + n - cached)
        cu_k.append(cu_k[-1] + n)
        max_q, max_k = max(max_q, n - cached), max(max_k, n)
        first_block = cached // block_size
        for i in range(first_block, seq.num_blocks):
            start = seq.block_table[i] * block_size
            count = block_size if i != seq.num_blocks - 1 else seq.last_block_num_tokens
            slot_mapping.extend(range(start, start + count))
    block_tables = None
    if cu_q[-1] < cu_k[-1]:
        width = max(len(seq.block_table) for seq in seqs)
        block_tables = [seq.block_table + [-1] * (width - len(seq.block_table)) for seq in seqs]
    return dict(input_ids=input_ids, cu_seqlens_q=cu_q, cu_seqlens_k=cu_k, max_seqlen_q=max_q,
                max_seqlen_k=max_k, slot_mapping=slot_mapping, block_tables=block_tables)


def decode_metadata(seqs, block_size: int) -> dict:
    input_ids = [seq.last_token for seq in seqs]
    context_lens = [len(seq) for seq in seqs]
    slot_mapping = [seq.block_table[-1] * block_size + seq.last_block_num_tokens - 1 for seq in seqs]
    width = max(len(seq.block_table) for seq in seqs)
    block_tables = [seq.block_table + [-1] * (width - len(seq.block_table)) for seq in seqs]
    return dict(input_ids=input_ids, context_lens=context_lens, slot_mapping=slot_mapping,
                block_tables=block_tables)
