"""Engine-side producers on the CPU: sequence block arithmetic, block manager (prefix hashes, ref counts),
scheduler (prefill-first, preemption, finish) and the per-step metadata vs the producers oracle."""
import random

import pytest
import xxhash
import numpy as np

import oracle
from minivllm_amd.engine.block_manager import BlockManager
from minivllm_amd.engine.llm_engine import LLMEngine
from minivllm_amd.engine.metadata import decode_metadata, prefill_metadata
from minivllm_amd.engine.scheduler import Scheduler
from minivllm_amd.engine.sequence import Sequence, SequenceStatus
from minivllm_amd.sampling_parameters import SamplingParams


def _seq(n, bs, start=0, **kw):
    return Sequence(list(range(start, start + n)), SamplingParams(**kw), bs)


def test_sequence_block_arithmetic_including_exact_multiples():
    s = _seq(8, 4)
    assert (s.num_blocks, s.last_block_num_tokens, s.block(1)) == (2, 4, [4, 5, 6, 7])
    s.append_token(99)
    assert (len(s), s.num_blocks, s.last_block_num_tokens, s.block(2), s.last_token) == (9, 3, 1, [99], 99)
    assert s.num_completion_tokens == 1 and s.completion_token_ids == [99]
    with pytest.raises(AssertionError):
        SamplingParams(temperature=0.0)


def test_compute_hash_is_chained_xxh64_of_int32_bytes():
    """XXH64 known answers: empty input with seed 0 is ef46db3751d8e999."""
    assert xxhash.xxh64(b"").intdigest() == 0xEF46DB3751D8E999
    toks = [1, 2, 3, 4]
    raw = np.array(toks, dtype=np.int32).tobytes()
    assert BlockManager.compute_hash(toks) == xxhash.xxh64(raw).intdigest()
    prefix = 0x0123456789ABCDEF
    assert BlockManager.compute_hash(toks, prefix) == xxhash.xxh64(prefix.to_bytes(8, "little") + raw).intdigest()
    assert BlockManager.compute_hash(toks, prefix) != BlockManager.compute_hash(toks)


def test_block_manager_allocate_free_and_prefix_sharing():
    bm = BlockManager(8, 4)
    a = _seq(10, 4)
    bm.allocate(a)
    assert len(a.block_table) == 3 and len(bm.free_block_ids) == 5 and a.num_cached_tokens == 0
    b = Sequence(list(range(8)) + [70, 71], SamplingParams(), 4)       # shares the first two full blocks
    bm.allocate(b)
    assert b.block_table[:2] == a.block_table[:2] and b.block_table[2] != a.block_table[2]
    assert b.num_cached_tokens == 8 and len(bm.free_block_ids) == 4
    assert bm.blocks[a.block_table[0]].ref_count == 2
    bm.deallocate(a)
    assert len(bm.free_block_ids) == 5 and bm.blocks[b.block_table[0]].ref_count == 1
    bm.deallocate(b)
    assert len(bm.free_block_ids) == 8 and not bm.used_block_ids
    c = _seq(8, 4)                                                      # cached hashes survive a free
    bm.allocate(c)
    assert c.num_cached_tokens == 4        # both blocks hit; the last one is handed back to be recomputed
    d = Sequence([5, 5, 5, 5, 4, 5, 6, 7], SamplingParams(), 4)         # same 2nd block tokens, other prefix: no hit
    bm.allocate(d)
    assert d.num_cached_tokens == 0


def test_block_manager_append_allocates_on_block_start_and_hashes_on_fill():
    bm = BlockManager(4, 4)
    s = _seq(4, 4)
    bm.allocate(s)
    assert len(s.block_table) == 1
    s.append_token(100)                       # 5 tokens: the new token starts block 1
    assert bm.can_append(s)
    bm.append(s)
    assert len(s.block_table) == 2 and bm.blocks[s.block_table[1]].hash == -1
    for t in (101, 102):
        s.append_token(t)
        bm.append(s)
    assert len(s.block_table) == 2
    s.append_token(103)                       # 8 tokens: this step fills block 1 -> it gets its chained hash
    bm.append(s)
    blk = bm.blocks[s.block_table[1]]
    assert blk.hash == BlockManager.compute_hash([100, 101, 102, 103], bm.blocks[s.block_table[0]].hash)
    bm2 = BlockManager(1, 4)
    t = _seq(4, 4)
    bm2.allocate(t)
    t.append_token(1)
    assert not bm2.can_append(t)


def _metadata_inputs(seqs):
    return [dict(num_tokens=len(s), num_cached_tokens=s.num_cached_tokens, block_table=list(s.block_table),
                 last_token=s.last_token) for s in seqs]


def test_metadata_matches_producers_oracle():
    rng = random.Random(0)
    for bs in (1, 4, 16):
        bm = BlockManager(200, bs)
        seqs = []
        for _ in range(5):
            s = _seq(rng.randint(1, 50), bs, start=rng.randint(0, 3))
            bm.allocate(s)
            seqs.append(s)
        got = prefill_metadata(seqs, bs, reuse_cached_kv=True)
        want = oracle.prefill_metadata_oracle(_metadata_inputs(seqs), bs)
        for key in ("cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "slot_mapping", "block_tables"):
            assert got[key] == want[key], (bs, key)
        full = prefill_metadata(seqs, bs, reuse_cached_kv=False)
        uncached = [dict(m, num_cached_tokens=0) for m in _metadata_inputs(seqs)]
        want_full = oracle.prefill_metadata_oracle(uncached, bs)
        assert full["slot_mapping"] == want_full["slot_mapping"] and full["cu_seqlens_q"] == want_full["cu_seqlens_k"]
        assert full["input_ids"] == [t for s in seqs for t in s.token_ids]
        for s in seqs:
            s.append_token(7)
            bm.append(s)
        got = decode_metadata(seqs, bs)
        want = oracle.decode_metadata_oracle(_metadata_inputs(seqs), bs)
        assert got == want


class FakeRunner:
    """Stands in for the model: returns a counter as the next token and records what it was asked to run."""

    def __init__(self):
        self.calls = []
        self.next = 1000

    def run(self, seqs, is_prefill):
        self.calls.append((is_prefill, [s.seq_id for s in seqs], [len(s) for s in seqs]))
        out = list(range(self.next, self.next + len(seqs)))
        self.next += len(seqs)
        return out


def test_engine_loop_prefill_first_then_decode_until_max_tokens():
    cfg = dict(max_num_sequences=2, max_num_batched_tokens=64, max_cached_blocks=16, block_size=4, eos=-1)
    runner = FakeRunner()
    eng = LLMEngine(cfg, model_runner=runner)
    prompts = [[1, 2, 3], [4, 5, 6, 7, 8], [9]]
    out = eng.generate(prompts, SamplingParams(temperature=0.6, max_tokens=4, ignore_eos=True))
    assert [len(t) for t in out["token_ids"]] == [4, 4, 4]
    # first two prompts admitted together (batch limit 2), then the third is prefilled before any decode
    assert runner.calls[0][0] is True and len(runner.calls[0][1]) == 2
    assert runner.calls[1][0] is True and len(runner.calls[1][1]) == 1
    assert all(c[0] is False for c in runner.calls[2:])
    # lengths advance by one per decode step (the sequence is really extended)
    first = runner.calls[0][1][0]
    lens = [c[2][c[1].index(first)] for c in runner.calls if first in c[1]]
    assert lens == [3, 4, 5, 6]
    assert eng.scheduler.is_finished() and len(eng.scheduler.block_manager.free_block_ids) == 16
    assert eng.stats["decode_tokens"] == 9 and eng.stats["prefill_tokens"] == 3 + 5 + 1


def test_scheduler_eos_and_token_budget_and_preemption():
    sch = Scheduler(max_num_sequences=8, max_num_batched_tokens=8, max_cached_blocks=3, block_size=4, eos=42)
    a, b = _seq(6, 4, max_tokens=10), _seq(4, 4, start=50, max_tokens=10)
    sch.add_sequence(a)
    sch.add_sequence(b)
    seqs, is_prefill = sch.schedule()
    assert is_prefill and seqs == [a]                 # 6 + 4 tokens exceed the 8-token budget
    sch.postprocess(seqs, [5])
    seqs, is_prefill = sch.schedule()
    assert is_prefill and seqs == [b]                 # waiting prompts go before decode
    sch.postprocess(seqs, [6])
    # 3 blocks in total: a holds 2, b holds 1; b's 5th token needs a block -> the tail sequence is preempted
    seqs, is_prefill = sch.schedule()
    assert not is_prefill and seqs == [a]
    assert b.status == SequenceStatus.WAITING and b.block_table == [] and sch.waiting[0] is b
    sch.postprocess(seqs, [42])                       # eos finishes a and frees its blocks
    assert a.is_finished and len(sch.block_manager.free_block_ids) == 3
    seqs, is_prefill = sch.schedule()
    assert is_prefill and seqs == [b] and len(b) == 5  # re-prefilled with prompt + generated token


def test_full_prefix_hit_still_leaves_one_block_to_compute():
    """A prompt made only of cached full blocks would have no query token in its prefill step; the allocator
    hands the last block back to be recomputed (it stays shared)."""
    from minivllm_amd.engine.block_manager import BlockManager
    from minivllm_amd.engine.metadata import prefill_metadata
    from minivllm_amd.engine.sequence import Sequence
    from minivllm_amd.sampling_parameters import SamplingParams
    bm = BlockManager(8, 4)
    sp = SamplingParams()
    first = Sequence(list(range(12)), sp, 4)
    bm.allocate(first)
    again = Sequence(list(range(8)), sp, 4)                       # blocks 0 and 1 of `first`
    bm.allocate(again)
    assert again.block_table == first.block_table[:2]
    assert again.num_cached_tokens == 4
    md = prefill_metadata([again], 4, reuse_cached_kv=True)
    assert md["input_ids"] == [4, 5, 6, 7] and md["cu_seqlens_q"] == [0, 4] and md["cu_seqlens_k"] == [0, 8]
    assert md["slot_mapping"] == [again.block_table[1] * 4 + i for i in range(4)]
    assert md["block_tables"] == [again.block_table]


def test_requests_longer_than_the_model_length_are_refused_at_admission():
    import pytest
    cfg = dict(max_num_sequences=2, max_num_batched_tokens=64, max_cached_blocks=16, block_size=4, eos=-1,
               max_position=32, max_model_length=24)
    eng = LLMEngine(cfg, model_runner=FakeRunner())
    eng.add_prompt(list(range(20)), SamplingParams(max_tokens=4))          # 24: fits exactly
    with pytest.raises(ValueError):
        eng.add_prompt(list(range(21)), SamplingParams(max_tokens=4))
    with pytest.raises(ValueError):
        eng.add_prompt([], SamplingParams(max_tokens=4))
    assert len(eng.scheduler.waiting) == 1


def test_decode_workspace_need_is_not_monotonic_and_the_runner_sizes_for_the_maximum():
    """The split-K scratch a decode call may use is not monotonic in the batch size (a smaller batch is cut into
    more partitions), so the model runner sizes one buffer for the maximum over its batch buckets before it
    captures any graph; every bucket then fits that buffer."""
    from minivllm_amd.layers.attention import decode_workspace_bytes
    hq, d, bs = 16, 128, 16
    for max_len in (4096, 8192):
        blocks = max_len // bs
        need = {b: decode_workspace_bytes(b, hq, d, blocks, bs) for b in [1, 2, 4, 8, 16, 32, 48, 64]}
        assert need[48] > need[64] > 0                 # 48 x 32 partitions against 64 x 16
        sized = max(need.values())
        assert all(n <= sized for n in need.values())


class FakeAsyncRunner(FakeRunner):
    """A runner that can launch decode steps ahead of their ids, as the model runner's hipGraph path does."""

    class Handle:
        def __init__(self, ids, log):
            self.ids, self.log = ids, log

        def wait(self):
            self.log.append("wait")
            return self.ids

    def __init__(self):
        super().__init__()
        self.log = []
        self.last = None

    def can_launch_decode(self, seqs):
        return True

    def continues_last_decode(self, seqs):
        return self.last is not None and self.last[0] == [s.seq_id for s in seqs] and \
            all(len(s) == n + 1 for s, n in zip(seqs, self.last[1]))

    def launch_decode(self, seqs):
        assert not any(s.is_finished for s in seqs), "a finished sequence has no blocks to build metadata from"
        assert all(len(s.block_table) == s.num_blocks for s in seqs), "every token of the step needs a cache slot"
        if not self.continues_last_decode(seqs):
            assert all(t >= 0 for s in seqs for t in s.token_ids), "a refill needs real last tokens"
        self.log.append("launch")
        ids = super().run(seqs, False)
        self.last = ([s.seq_id for s in seqs], [len(s) for s in seqs])
        return self.Handle(ids, self.log)

    def run(self, seqs, is_prefill):
        assert all(t >= 0 for s in seqs for t in s.token_ids), "a synchronous step needs real token ids"
        assert not any(s.is_finished for s in seqs) and all(len(s.block_table) == s.num_blocks for s in seqs)
        self.last = None
        self.log.append("run")
        return super().run(seqs, is_prefill)


def test_decode_steps_launched_ahead_of_their_ids_give_the_same_run():
    """async_decode: decode steps of sequences that ignore EOS are launched before the previous step's ids reach
    the host.  Tokens, finish order, freed blocks and the hashes of the blocks that filled up on the way must equal
    the synchronous engine's; every launch but the first of a batch happens before the wait for the step before."""
    cfg = dict(max_num_sequences=3, max_num_batched_tokens=64, max_cached_blocks=24, block_size=4, eos=-1,
               max_position=64)
    prompts = [[1, 2, 3], [4, 5, 6, 7, 8], [9], [10, 11, 12, 13, 14, 15, 16]]
    sp = SamplingParams(temperature=0.6, max_tokens=9, ignore_eos=True)
    engines = {}
    for mode in (False, True):
        runner = FakeAsyncRunner()
        eng = LLMEngine(dict(cfg, async_decode=mode), model_runner=runner)
        out = eng.generate(prompts, sp)["token_ids"]
        engines[mode] = (out, eng, runner)
        assert [len(t) for t in out] == [9] * 4 and all(t >= 0 for seq in out for t in seq)
        assert eng.scheduler.is_finished() and eng.pending is None
        assert len(eng.scheduler.block_manager.free_block_ids) == 24
    assert engines[True][0] == engines[False][0]
    hashes = [set(engines[mode][1].scheduler.block_manager.hash_to_block_id) for mode in (True, False)]
    assert hashes[0] == hashes[1] and len(hashes[0]) >= 8
    log = engines[True][2].log
    assert "wait" in log and "launch" in log and "wait" not in engines[False][2].log
    # steady state: launch(t + 1) comes before wait(t)
    assert "launch launch launch" not in " ".join(log)             # one step outstanding besides the one just launched
    assert sum(1 for a, b in zip(log, log[1:]) if a == "launch" and b == "wait") >= 6


class FakeFunctionRunner(FakeAsyncRunner):
    """Ids that depend only on (sequence, position), so a run does not depend on which rows were computed for
    nothing; ``eos_at`` maps a sequence's position in the batch order to the length at which it emits EOS."""

    def __init__(self, eos, eos_at):
        super().__init__()
        self.eos, self.eos_at, self.order = eos, eos_at, {}

    def _ids(self, seqs):
        out = []
        for s in seqs:
            k = self.order.setdefault(s.seq_id, len(self.order))
            out.append(self.eos if self.eos_at.get(k) == len(s) else 2000 + 37 * k + len(s))
        return out

    def launch_decode(self, seqs):
        assert not any(s.is_finished for s in seqs), "a finished sequence has no blocks to build metadata from"
        assert all(len(s.block_table) == s.num_blocks for s in seqs), "every token of the step needs a cache slot"
        if not self.continues_last_decode(seqs):
            assert all(t >= 0 for s in seqs for t in s.token_ids), "a refill needs real last tokens"
        self.log.append("launch")
        self.calls.append((False, [s.seq_id for s in seqs], [len(s) for s in seqs]))
        self.last = ([s.seq_id for s in seqs], [len(s) for s in seqs])
        return self.Handle(self._ids(seqs), self.log)

    def run(self, seqs, is_prefill):
        assert all(t >= 0 for s in seqs for t in s.token_ids), "a synchronous step needs real token ids"
        assert not any(s.is_finished for s in seqs) and all(len(s.block_table) == s.num_blocks for s in seqs)
        self.last = None
        self.log.append("run")
        self.calls.append((is_prefill, [s.seq_id for s in seqs], [len(s) for s in seqs]))
        return self._ids(seqs)


def test_sequences_that_stop_at_eos_also_run_ahead_and_end_one_commit_late():
    """Decode steps are launched ahead of their ids also when a sequence may stop at EOS: the EOS is seen when the
    ids arrive, one step late, the sequence ends there, and the row the next step computed for it is dropped.  Tokens,
    finish order and freed blocks equal the synchronous engine's; sequences that end by EOS, by count, at a block
    boundary and in the step right after their prefill are all in the batch."""
    eos = 7
    cfg = dict(max_num_sequences=3, max_num_batched_tokens=64, max_cached_blocks=24, block_size=4, eos=eos,
               max_position=64)
    prompts = [[1, 2, 3], [4, 5, 6, 8, 9], [10], [11, 12, 13, 14, 15, 16, 17], [18, 19]]
    # sequence k emits EOS when it is eos_at[k] tokens long: 0 in its second decode step, 1 as the token that opens a
    # new block (length 8), 2 never (ends by count), 3 with its first sampled token (the prefill's), 4 at length 9
    eos_at = {0: 5, 1: 8, 3: 7, 4: 9}
    sp = SamplingParams(temperature=0.6, max_tokens=10, ignore_eos=False)
    runs = {}
    for mode in (False, True):
        runner = FakeFunctionRunner(eos, eos_at)
        eng = LLMEngine(dict(cfg, async_decode=mode), model_runner=runner)
        order = []
        for p in prompts:
            eng.add_prompt(p, sp)
        while not eng.scheduler.is_finished() or eng.pending is not None:
            finished, _, _ = eng.step()
            order += [sid for sid, _ in finished]
        runs[mode] = (order, eng, runner)
        assert eng.pending is None and len(eng.scheduler.block_manager.free_block_ids) == 24
    tokens = {}
    for mode in (False, True):
        runner = FakeFunctionRunner(eos, eos_at)
        eng = LLMEngine(dict(cfg, async_decode=mode), model_runner=runner)
        tokens[mode] = eng.generate(prompts, sp)["token_ids"]
    assert tokens[True] == tokens[False]
    lengths = [len(t) for t in tokens[True]]
    assert lengths == [3, 4, 10, 1, 8] and [t[-1] for t in tokens[True]].count(eos) == 4
    assert all(eos not in t[:-1] for t in tokens[True])                # nothing is generated past an EOS
    assert all(len(runs[m][0]) == 5 and len(set(runs[m][0])) == 5 for m in (True, False))   # each reported once
    log = runs[True][2].log
    assert sum(1 for a, b in zip(log, log[1:]) if a == "launch" and b == "wait") >= 4  # steps did run ahead


@pytest.mark.parametrize("shared_prefixes", [False, True])
def test_run_ahead_equals_waiting_engine_on_random_schedules(shared_prefixes):
    """Property: for random prompts (distinct, or cut from one stem so that prefix blocks are shared), EOS positions,
    token limits, batch limits and block sizes (preemption when the pool is small included) the engine that launches
    decode steps ahead of their ids returns the same tokens per sequence as the one that waits, reports every sequence
    once, and leaves the block manager empty: every block free, no reference, no hash waiting for an id."""
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=300, deadline=None, derandomize=True)
    @given(st.data())
    def check(data):
        n = data.draw(st.integers(1, 7))
        if shared_prefixes:
            stem = [data.draw(st.integers(1, 3)) for _ in range(20)]
            prompts = []
            for _ in range(n):
                keep = data.draw(st.integers(0, 16))
                tail = [50 + data.draw(st.integers(0, 2)) for _ in range(data.draw(st.integers(0 if keep else 1, 6)))]
                prompts.append(stem[:keep] + tail)
        else:
            prompts = [list(range(100 * i + 1, 100 * i + 1 + data.draw(st.integers(1, 14)))) for i in range(n)]
        max_tokens = data.draw(st.integers(1, 12))
        block_size = data.draw(st.sampled_from([2, 4, 8]))
        longest = max(map(len, prompts)) + max_tokens
        blocks = data.draw(st.integers(-(-longest // block_size) + 1, 40))      # at least one sequence always fits
        cfg = dict(max_num_sequences=data.draw(st.integers(1, 4)), max_num_batched_tokens=64, max_cached_blocks=blocks,
                   block_size=block_size, eos=7, max_position=64)
        eos_at = {k: data.draw(st.integers(len(p), len(p) + max_tokens + 2)) for k, p in enumerate(prompts)
                  if data.draw(st.booleans())}
        sp = SamplingParams(temperature=0.6, max_tokens=max_tokens, ignore_eos=data.draw(st.booleans()))
        outs = []
        for ahead in (True, False):
            eng = LLMEngine(dict(cfg, async_decode=ahead), model_runner=FakeFunctionRunner(7, eos_at))
            for p in prompts:
                eng.add_prompt(p, sp)
            reported = []
            steps = 0
            while not eng.scheduler.is_finished() or eng.pending is not None:
                finished, _, _ = eng.step()
                reported += finished
                steps += 1
                assert steps < 3000
            bm = eng.scheduler.block_manager
            assert len(reported) == n and len({sid for sid, _ in reported}) == n
            assert len(bm.free_block_ids) == blocks and not bm.used_block_ids and eng.pending is None
            assert all(b.ref_count == 0 for b in bm.blocks) and not bm.deferred
            assert all(t >= 0 for b in bm.blocks if b.hash != -1 for t in b.token_ids)    # no hash over a placeholder
            outs.append([toks for _, toks in sorted(reported)])
        assert outs[0] == outs[1]
        for toks in outs[0]:
            assert 1 <= len(toks) <= max_tokens and all(t >= 0 for t in toks)
            if not sp.ignore_eos:
                assert 7 not in toks[:-1]

    check()


def test_eos_of_a_sequence_preempted_while_its_id_was_on_the_way():
    """A sequence whose step was launched, that is then preempted by the scheduling of the next step (the pool is
    full) and whose id turns out to be its EOS: the commit ends it from the waiting queue, its blocks having been
    returned by the preemption.  (Found by the random-schedule property above: three one-token prompts, blocks of
    two tokens, a pool of six.)"""
    cfg = dict(max_num_sequences=3, max_num_batched_tokens=64, max_cached_blocks=6, block_size=2, eos=7,
               max_position=64)
    prompts = [[1], [101], [201]]
    sp = SamplingParams(temperature=0.6, max_tokens=5, ignore_eos=False)
    outs = []
    for ahead in (True, False):
        eng = LLMEngine(dict(cfg, async_decode=ahead), model_runner=FakeFunctionRunner(7, {2: 4}))
        for p in prompts:
            eng.add_prompt(p, sp)
        reported = []
        for _ in range(200):
            if eng.scheduler.is_finished() and eng.pending is None:
                break
            finished, _, _ = eng.step()
            reported += finished
        assert len(reported) == 3 and len(eng.scheduler.block_manager.free_block_ids) == 6
        outs.append([toks for _, toks in sorted(reported)])
    assert outs[0] == outs[1]


def test_a_reused_block_is_not_shared_through_its_old_hash():
    """A freed block keeps its hash so that a later prompt can share it.  Once the block is taken for something else,
    that hash must stop leading to it: here block 2 first ends the prefix [2, 1, 1], is freed, then holds the third
    token of [3, 1, 1], the same token 1, and a new [2, 1, 1] must not share it (its K/V were computed behind another
    prefix; the reference's check compares the block's own tokens only, block_manager.py:72-86).  Found by the random
    operation sequences below."""
    bm = BlockManager(7, 1)
    a = Sequence([2, 1, 1], SamplingParams(), 1)
    bm.allocate(a)
    first = list(a.block_table)
    bm.deallocate(a)
    b, c = Sequence([3], SamplingParams(), 1), Sequence([1, 1], SamplingParams(), 1)
    bm.allocate(b)
    bm.allocate(c)
    for _ in range(2):
        b.append_token(1)
        bm.append(b)
    assert b.block_table[2] == first[2]                      # the old third block of [2, 1, 1] now belongs to [3, 1, 1]
    bm.deallocate(c)
    d = Sequence([2, 1, 1], SamplingParams(), 1)
    bm.allocate(d)
    assert d.block_table[:2] == first[:2] and d.num_cached_tokens == 2      # the first two blocks are still shareable
    assert d.block_table[2] != b.block_table[2] and len(set(d.block_table)) == 3


def test_block_manager_invariants_under_random_operations():
    """Random allocate / append / free sequences over prompts cut from one stem (so that prefixes are shared and freed
    blocks are found again): reference counts equal the number of tables a block is in, free and used blocks partition
    the pool, no table holds a block twice, cached prefixes hold the sequence's own tokens, and two sequences share a
    block only behind equal prefixes."""
    from hypothesis import given, settings, strategies as st

    def invariants(bm, live, bs):
        counts = {}
        for s in live:
            assert len(s.block_table) == s.num_blocks and len(set(s.block_table)) == len(s.block_table)
            for b in s.block_table:
                counts[b] = counts.get(b, 0) + 1
            assert s.num_cached_tokens % bs == 0 and 0 <= s.num_cached_tokens <= max(len(s) - 1, 0)
            for i in range(s.num_cached_tokens // bs):
                assert bm.blocks[s.block_table[i]].token_ids == s.block(i)
            h = -1
            for i in range(len(s) // bs):                       # a full block's hash, if it has one, is its prefix chain's
                h = BlockManager.compute_hash(s.block(i), h)
                if all(t >= 0 for t in s.token_ids[:(i + 1) * bs]):
                    assert bm.blocks[s.block_table[i]].hash in (-1, h)
        assert all(b.ref_count == counts.get(b.block_id, 0) for b in bm.blocks)
        assert set(bm.free_block_ids).isdisjoint(bm.used_block_ids) and bm.used_block_ids == set(counts)
        assert len(bm.free_block_ids) + len(bm.used_block_ids) == len(bm.blocks)
        for a in live:
            for c in live:
                for i, (x, y) in enumerate(zip(a.block_table, c.block_table)):
                    assert x != y or a.token_ids[:(i + 1) * bs] == c.token_ids[:(i + 1) * bs]

    @settings(max_examples=400, deadline=None, derandomize=True)
    @given(st.data())
    def check(data):
        bs = data.draw(st.sampled_from([1, 2, 4]))
        nblocks = data.draw(st.integers(4, 24))
        bm = BlockManager(nblocks, bs)
        stem = [data.draw(st.integers(1, 2)) for _ in range(16)]
        live = []
        for _ in range(data.draw(st.integers(1, 40))):
            op = data.draw(st.sampled_from(["alloc", "alloc", "append", "append", "append", "free"]))
            if op == "alloc":
                keep = data.draw(st.integers(0, 12))
                tail = [data.draw(st.integers(1, 3)) for _ in range(data.draw(st.integers(0 if keep else 1, 5)))]
                s = Sequence(stem[:keep] + tail, SamplingParams(), bs)
                if bm.can_allocate(s):
                    bm.allocate(s)
                    live.append(s)
            elif op == "append" and live:
                s = live[data.draw(st.integers(0, len(live) - 1))]
                if len(bm.free_block_ids) >= 1:                 # the token may open a block
                    s.append_token(data.draw(st.sampled_from([1, 2, 3, -1])))      # -1: an id still on its way
                    bm.append(s)
                    if s.token_ids[-1] < 0:
                        s.token_ids[-1] = s.last_token = data.draw(st.integers(1, 3))
                        bm.hash_deferred_blocks()
            elif op == "free" and live:
                bm.deallocate(live.pop(data.draw(st.integers(0, len(live) - 1))))
            invariants(bm, live, bs)
        for s in live:
            bm.deallocate(s)
        invariants(bm, [], bs)
        assert len(bm.free_block_ids) == nblocks

    check()


def test_requests_the_scheduler_could_never_place_are_refused():
    """A prompt that no step's token budget can take, or whose tokens need more blocks than the pool has, would wait for
    ever (also after a preemption, when it is prefilled again at its full length): ``add_prompt`` raises instead."""
    cfg = dict(max_num_sequences=2, max_num_batched_tokens=16, max_cached_blocks=3, block_size=4, eos=-1, max_position=64)
    eng = LLMEngine(cfg, model_runner=FakeRunner())
    sp = SamplingParams(temperature=0.6, max_tokens=4, ignore_eos=True)
    with pytest.raises(ValueError, match="max_num_batched_tokens"):
        eng.add_prompt(list(range(1, 15)), sp)                 # 14 + 4 - 1 = 17 tokens in a step of 16
    with pytest.raises(ValueError, match="blocks"):
        eng.add_prompt(list(range(1, 11)), sp)                 # 13 tokens = 4 blocks of 4, the pool has 3
    eng.add_prompt(list(range(1, 10)), sp)                     # 12 tokens = 3 blocks: fits exactly
    out = eng.generate([], sp)
    assert [len(t) for t in out["token_ids"]] == [4] and len(eng.scheduler.block_manager.free_block_ids) == 3
