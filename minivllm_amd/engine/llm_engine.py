"""Engine front end: queue prompts, step until done, report tokens/s
(src/myvllm/engine/llm_engine.py:13-88).  Prompts are lists of token ids (a tokenizer, if any, is the
caller's business: the reference fetches one by name over the network)."""
from __future__ import annotations

import time

from minivllm_amd.engine.model_runner import ModelRunner
from minivllm_amd.engine.scheduler import Scheduler
from minivllm_amd.engine.sequence import Sequence
from minivllm_amd.sampling_parameters import SamplingParams


class LLMEngine:
    def __init__(self, config: dict, model_runner=None):
        self.block_size = config.get("block_size", 256)
        self.scheduler = Scheduler(
            max_num_sequences=config.get("max_num_sequences", 16),
            max_num_batched_tokens=config.get("max_num_batched_tokens", 1024),
            max_cached_blocks=config.get("max_cached_blocks", 1024),
            block_size=self.block_size,
            eos=config.get("eos", 50256))
        self.model_runner = model_runner if model_runner is not None else ModelRunner(config)
        # longest sequence (prompt + new tokens) the rotary table and the graph's block-table buffer are sized for
        self.max_model_length = min(config.get("max_model_length", config.get("max_position", 4096)),
                                    config.get("max_position", 4096))
        self.stats = {"prefill_tokens": 0, "decode_tokens": 0, "prefill_s": 0.0, "decode_s": 0.0, "steps": 0}

    def add_prompt(self, prompt_token_ids: list[int], sampling_params: SamplingParams) -> None:
        """Queue a prompt.  A request that could outgrow ``max_model_length`` / ``max_position`` is refused here:
        the reference's demo exceeds its own limit silently (main.py:35,38,49) and would index the rotary table
        out of range (rotary_embedding.py:78)."""
        if not prompt_token_ids:
            raise ValueError("empty prompt")
        longest = len(prompt_token_ids) + sampling_params.max_tokens
        if longest > self.max_model_length:
            raise ValueError(f"prompt of {len(prompt_token_ids)} tokens + max_tokens {sampling_params.max_tokens} "
                             f"exceeds max_model_length / max_position {self.max_model_length}")
        self.scheduler.add_sequence(Sequence(prompt_token_ids, sampling_params, self.block_size))

    def step(self):
        """One schedule -> run -> postprocess round.  Always a 3-tuple (finished, processed tokens, is_prefill)."""
        seqs, is_prefill = self.scheduler.schedule()
        if not seqs:
            return [], 0, is_prefill
        token_ids = self.model_runner.run(seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        finished = [(seq.seq_id, seq.completion_token_ids) for seq in seqs if seq.is_finished]
        processed = sum(len(seq) - 1 for seq in seqs) if is_prefill else len(seqs)
        return finished, processed, is_prefill

    def generate(self, prompts: list[list[int]], sampling_params: SamplingParams, verbose: bool = False) -> dict:
        for prompt in prompts:
            self.add_prompt(prompt, sampling_params)
        done = {}
        while not self.scheduler.is_finished():
            t0 = time.perf_counter()
            finished, processed, is_prefill = self.step()
            dt = time.perf_counter() - t0
            kind = "prefill" if is_prefill else "decode"
            self.stats[kind + "_tokens"] += processed
            self.stats[kind + "_s"] += dt
            self.stats["steps"] += 1
            if verbose:
                print(f"{processed} tokens, {processed / (dt + 1e-10):.1f} tokens/sec during {kind}")
            done.update(finished)
        return {"token_ids": [done[k] for k in sorted(done)]}
