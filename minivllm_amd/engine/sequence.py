"""Per-request state and block arithmetic (src/myvllm/engine/sequence.py:14-104).

Differences from the reference, on purpose: ``block_size`` is per instance (the
reference hard-codes 256 on the class, sequence.py:15, while the engine config
carries its own value) and ``last_block_num_tokens`` is the number of tokens
held by the final block, in 1..block_size (the reference's expression is 0 on
exact multiples, which drops slots in prepare_prefill/prepare_decode).
"""
from __future__ import annotations

from copy import copy
from enum import Enum, auto
from itertools import count

from minivllm_amd.sampling_parameters import SamplingParams


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class Sequence:
    counter = count()

    def __init__(self, token_ids: list[int], sampling_params: SamplingParams | None = None, block_size: int = 256):
        sampling_params = sampling_params if sampling_params is not None else SamplingParams()
        if not token_ids:
            raise ValueError("a sequence needs at least one prompt token")
        self.block_size = block_size
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = copy(token_ids)
        self.last_token = self.token_ids[-1]
        self.num_tokens = len(self.token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_cached_tokens = 0
        self.block_table: list[int] = []
        self.temperature = sampling_params.temperature
        self.max_tokens = sampling_params.max_tokens
        self.ignore_eos = sampling_params.ignore_eos

    def __len__(self):
        return self.num_tokens

    def __getitem__(self, idx):
        return self.token_ids[idx]

    @property
    def is_finished(self):
        return self.status == SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self):
        return self.num_tokens - self.num_prompt_tokens

    @property
    def prompt_token_ids(self):
        return self.token_ids[:self.num_prompt_tokens]

    @property
    def completion_token_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def num_cached_blocks(self):
        return -(-self.num_cached_tokens // self.block_size)

    @property
    def num_blocks(self):
        return -(-self.num_tokens // self.block_size)

    @property
    def last_block_num_tokens(self):
        return self.num_tokens - (self.num_blocks - 1) * self.block_size

    def block(self, i):
        assert 0 <= i < self.num_blocks, f"Block index {i} out of range [0, {self.num_blocks})"
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def append_token(self, token_id):
        self.token_ids.append(token_id)
        self.last_token = token_id
        self.num_tokens += 1
