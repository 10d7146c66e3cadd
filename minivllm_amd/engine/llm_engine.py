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
        self.async_decode = config.get("async_decode", True)
        self.pending = None          # (ids on their way, placeholders to fill, sequences that step finished)
        self.stats = {"prefill_tokens": 0, "decode_tokens": 0, "prefill_s": 0.0, "decode_s": 0.0, "steps": 0}

    def add_prompt(self, prompt_token_ids: list[int], sampling_params: SamplingParams) -> None:
        """Queue a prompt.  A request that could outgrow ``max_model_length`` / ``max_position`` is refused here:
        the reference's demo exceeds its own limit silently (main.py:35,38,49) and would index the rotary table
        out of range (rotary_embedding.py:78).  So is one that no step's token budget or the block pool can hold."""
        if not prompt_token_ids:
            raise ValueError("empty prompt")
        longest = len(prompt_token_ids) + sampling_params.max_tokens
        if longest > self.max_model_length:
            raise ValueError(f"prompt of {len(prompt_token_ids)} tokens + max_tokens {sampling_params.max_tokens} "
                             f"exceeds max_model_length / max_position {self.max_model_length}")
        # what the scheduler could never place would wait for ever (the reference's generate loop spins on it,
        # llm_engine.py:62-75): a sequence is re-admitted as a whole after a preemption, so its full length must fit
        # the token budget of a step, and its blocks the pool
        slots = longest - 1                                     # the last sampled token is never fed back
        if slots > self.scheduler.max_num_batched_tokens:
            raise ValueError(f"prompt + max_tokens - 1 = {slots} tokens exceed max_num_batched_tokens "
                             f"{self.scheduler.max_num_batched_tokens}")
        pool = len(self.scheduler.block_manager.blocks)
        if -(-slots // self.block_size) > pool:
            raise ValueError(f"{slots} tokens need {-(-slots // self.block_size)} blocks of {self.block_size}, the pool has {pool}")
        self.scheduler.add_sequence(Sequence(prompt_token_ids, sampling_params, self.block_size))

    def step(self):
        """One schedule -> run -> postprocess round.  Always a 3-tuple (finished, processed tokens, is_prefill).

        With ``async_decode`` (default) a decode step is launched without waiting for the token ids of the step
        before: lengths, block tables and the finish-by-count do not depend on them, the next step's input ids are
        taken from the device, and the host schedules and launches step t + 1 while the GPU runs step t.  Such a
        step's ids are committed, and its finished sequences reported, one ``step`` later (or by ``flush``).  A
        sequence whose id turns out to be its EOS ends at that commit; the row the step launched in the meantime
        computed for it is dropped (its cache slot belongs to blocks that are freed with the sequence).  Everything
        that needs real ids (a prefill, a batch that changed) commits first."""
        finished = []
        if self.pending is not None and self.scheduler.waiting:
            finished += self.flush()                   # admission hashes prompt blocks: ids must be real
        seqs, is_prefill = self.scheduler.schedule()
        if not seqs:
            return finished + self.flush(), 0, is_prefill
        runner = self.model_runner
        if (self.async_decode and not is_prefill and hasattr(runner, "launch_decode")
                and runner.can_launch_decode(seqs)):
            if not runner.continues_last_decode(seqs):
                finished += self.flush()               # the buffers are refilled from the last tokens
                # an id that just arrived may have been a scheduled sequence's EOS: it has ended and given its
                # blocks (the one this step's scheduling appended included) back
                seqs = [seq for seq in seqs if not seq.is_finished]
                if not seqs:
                    return finished, 0, False
            handle = runner.launch_decode(seqs)
            finished += self.flush()                   # the step before this one, while the GPU runs this one
            slots, done = self.scheduler.postprocess_provisional(seqs)
            self.pending = (handle, slots, done)
            return finished, sum(slot is not None for slot in slots), False
        finished += self.flush()
        if not is_prefill:                             # as above: a scheduled sequence may just have ended
            seqs = [seq for seq in seqs if not seq.is_finished]
            if not seqs:
                return finished, 0, False
        token_ids = runner.run(seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        finished += [(seq.seq_id, seq.completion_token_ids) for seq in seqs if seq.is_finished]
        processed = sum(len(seq) - 1 for seq in seqs) if is_prefill else len(seqs)
        return finished, processed, is_prefill

    def flush(self):
        """Commit the token ids of a decode step that was launched ahead; returns the sequences it finished."""
        if self.pending is None:
            return []
        handle, slots, done = self.pending
        self.pending = None
        ended = self.scheduler.commit(slots, handle.wait())
        return [(seq.seq_id, seq.completion_token_ids) for seq in done + ended]

    def generate(self, prompts: list[list[int]], sampling_params: SamplingParams, verbose: bool = False) -> dict:
        for prompt in prompts:
            self.add_prompt(prompt, sampling_params)
        done = {}
        while not self.scheduler.is_finished() or self.pending is not None:
            t0 = time.perf_counter()
            finished, processed, is_prefill = self.step()
            dt = time.perf_counter() - t0
            kind = "prefill" if is_prefill else "decode"
            self.stats[kind + "_tokens"] += processed
            self.stats[kind + "_s"] += dt
            self.stats["steps"] += 1 if processed else 0
            if verbose:
                print(f"{processed} tokens, {processed / (dt + 1e-10):.1f} tokens/sec during {kind}")
            done.update(finished)
        return {"token_ids": [done[k] for k in sorted(done)]}
