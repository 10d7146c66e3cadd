"""Prefill-first continuous batching (src/myvllm/engine/scheduler.py:6-82).

Intended semantics where the reference is broken: limits are checked before a
sequence is popped from ``running`` (the reference pops then breaks, losing
it, scheduler.py:45,54-55), and ``postprocess`` advances the sequence with
``append_token`` (the reference appends to ``token_ids`` only, so lengths never
move, scheduler.py:78-79).
"""
from __future__ import annotations

from collections import deque

from minivllm_amd.engine.block_manager import BlockManager
from minivllm_amd.engine.sequence import Sequence, SequenceStatus


class Scheduler:
    def __init__(self, max_num_sequences: int, max_num_batched_tokens: int, max_cached_blocks: int,
                 block_size: int, eos: int):
        self.block_manager = BlockManager(max_cached_blocks, block_size)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_num_sequences = max_num_sequences
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        self.eos = eos

    def is_finished(self):
        return not self.waiting and not self.running

    def add_sequence(self, sequence: Sequence):
        self.waiting.append(sequence)

    def schedule(self) -> tuple[list[Sequence], bool]:
        scheduled: list[Sequence] = []
        num_tokens = 0
        # prefill: admit waiting sequences while blocks, token budget and batch slots last
        while self.waiting and len(scheduled) < self.max_num_sequences:
            seq = self.waiting[0]
            if len(seq) + num_tokens > self.max_num_batched_tokens or not self.block_manager.can_allocate(seq):
                break
            self.waiting.popleft()
            self.block_manager.allocate(seq)
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
            scheduled.append(seq)
            num_tokens += len(seq)
        if scheduled:
            return scheduled, True

        # decode: one token for each running sequence, preempting from the tail when blocks run out
        while self.running and len(scheduled) < self.max_num_sequences and num_tokens < self.max_num_batched_tokens:
            seq = self.running.popleft()
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    break
            else:
                self.block_manager.append(seq)
                scheduled.append(seq)
                num_tokens += 1
        if scheduled:
            self.running.extendleft(reversed(scheduled))
        return scheduled, False

    def preempt(self, seq: Sequence) -> None:
        self.block_manager.deallocate(seq)
        seq.status = SequenceStatus.WAITING
        self.waiting.appendleft(seq)

    PLACEHOLDER = -1        # stands for a sampled token whose id has not reached the host yet

    def postprocess_provisional(self, seqs: list[Sequence]):
        """``postprocess`` for a decode step whose token ids are still on the device: every sequence grows by a
        placeholder and finishes by count.  A sequence that has ended in the meantime (the ids of the step before
        arrived after this step was launched and held its EOS) is skipped: its row of this step is computed for
        nothing.  Returns the slots for ``commit``, one per row ((sequence, index of the placeholder) or None), and
        the sequences this step finished by count."""
        slots, done = [], []
        for seq in seqs:
            if seq.is_finished:
                slots.append(None)
                continue
            seq.append_token(self.PLACEHOLDER)
            slots.append((seq, seq.num_tokens - 1))
            if seq.num_completion_tokens >= seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
                done.append(seq)
        return slots, done

    def commit(self, slots: list, token_ids: list[int]) -> list[Sequence]:
        """The ids of a provisional step have arrived: replace the placeholders, end the sequences whose id is their
        EOS (one step late: the step launched in the meantime has computed a row for them that is dropped), then give
        the blocks that filled up in the meantime their hashes.  Returns the sequences ended here."""
        ended = []
        for slot, token_id in zip(slots, token_ids):
            if slot is None:
                continue
            seq, index = slot
            token_id = int(token_id)
            seq.token_ids[index] = token_id
            if index == seq.num_tokens - 1:
                seq.last_token = token_id
            if not seq.ignore_eos and token_id == self.eos and not seq.is_finished:
                if seq.status == SequenceStatus.WAITING:
                    # preempted by the scheduling of the step launched in the meantime: its blocks are back already
                    self.waiting.remove(seq)
                else:
                    self.block_manager.deallocate(seq)
                    self.running.remove(seq)
                seq.status = SequenceStatus.FINISHED
                ended.append(seq)
        self.block_manager.hash_deferred_blocks()
        return ended

    def postprocess(self, seqs: list[Sequence], token_ids: list[int]) -> None:
        for seq, token_id in zip(seqs, token_ids):
            seq.append_token(int(token_id))
            if (not seq.ignore_eos and token_id == self.eos) or seq.num_completion_tokens >= seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
