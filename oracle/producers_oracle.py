"""CPU restatement of the engine-side metadata producers (pure integer work).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

A sequence is described by plain values: ``num_tokens``, ``num_cached_tokens``,
``block_table`` (list of physical block ids) and, for decode, ``last_token``.
Deviation from the reference, on purpose: ``Sequence.last_block_num_tokens``
(sequence.py:70-72) evaluates to 0 when num_tokens is an exact multiple of
block_size, which makes the reference drop the final block's slots in prefill
(model_runner.py:207-208) and point the decode slot one row before the block
(:239).  The intended value -- tokens held by the final block, in 1..bs -- is
used here, so every token owns exactly one slot.

Pinned in tests/test_oracle_pins.py by the reference's own worked example
(model_runner.py:174-179: cu_seqlens_q = [0,3,5,9]), by hand-worked slot
arithmetic and by hypothesis properties (unique slots inside owned blocks).
"""
from __future__ import annotations


def _ceil_div(a, b):
    return -(-a // b)


def prefill_metadata_oracle(seqs, block_size):
    """src/myvllm/engine/model_runner.py:180-227.

    ``seqs``: list of dicts with keys num_tokens, num_cached_tokens, block_table.
    Returns dict(cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
    slot_mapping, block_tables-or-None, token_ranges) with plain lists.
    """
    cu_q, cu_k, slots, ranges = [0], [0], [], []
    lens_q, lens_k = [], []
    for s in seqs:
        n, cached, table = s["num_tokens"], s["num_cached_tokens"], s["block_table"]
        ranges.append((cached, n))                       # input_ids = tokens[cached:]   (:194)
        lens_q.append(n - cached)                        # (:195)
        lens_k.append(n)                                 # (:196)
        cu_q.append(cu_q[-1] + lens_q[-1])
        cu_k.append(cu_k[-1] + lens_k[-1])
        num_blocks = _ceil_div(n, block_size)
        cached_blocks = _ceil_div(cached, block_size)
        last_fill = n - (num_blocks - 1) * block_size    # tokens in the final block, 1..bs
        for i, blk in enumerate(table[cached_blocks:]):  # (:199-208)
            if cached_blocks + i != num_blocks - 1:
                count = block_size
            else:
                count = last_fill
            slots.extend(range(blk * block_size, blk * block_size + count))
    tables = None
    if cu_q[-1] < cu_k[-1]:                              # only when a prefix was cached (:209-215)
        width = max(len(s["block_table"]) for s in seqs)
        tables = [list(s["block_table"]) + [-1] * (width - len(s["block_table"])) for s in seqs]
    return dict(cu_seqlens_q=cu_q, cu_seqlens_k=cu_k,
                max_seqlen_q=max(lens_q), max_seqlen_k=max(lens_k),
                slot_mapping=slots, block_tables=tables, token_ranges=ranges)


def decode_metadata_oracle(seqs, block_size):
    """src/myvllm/engine/model_runner.py:231-256.

    ``seqs``: list of dicts with keys num_tokens, block_table, last_token.
    slot = block_table[-1]*bs + last_block_num_tokens - 1 (:239) where
    last_block_num_tokens follows sequence.py:70-72.
    """
    input_ids, ctx, slots = [], [], []
    for s in seqs:
        n, table = s["num_tokens"], s["block_table"]
        last_fill = n - (_ceil_div(n, block_size) - 1) * block_size
        input_ids.append(s["last_token"])
        ctx.append(n)
        slots.append(table[-1] * block_size + last_fill - 1)
    width = max(len(s["block_table"]) for s in seqs)
    tables = [list(s["block_table"]) + [-1] * (width - len(s["block_table"])) for s in seqs]
    return dict(input_ids=input_ids, context_lens=ctx, slot_mapping=slots, block_tables=tables)
