"""Model runner: builds the model and the paged KV pool, turns scheduled sequences into the per-step
``Context`` and runs one engine step (src/myvllm/engine/model_runner.py:14-308, single GPU, no process
group, no SHM workers).

Config keys (one set of names; the reference's runner and engine disagree on two of them): model keys
``vocab_size hidden_size num_layers num_heads num_kv_heads head_dim intermediate_size base
rms_norm_epsilon qkv_bias ffn_bias scale tie_word_embeddings max_position``; engine keys ``block_size
max_cached_blocks max_num_sequences max_num_batched_tokens dtype kv_cache_dtype seed``; ``linear_small_rows`` (default
64): projections of at most that many rows, a decode step, run as the single-launch ``linear_small_m``, the gate/up
projection with SiluAndMul as its epilogue (0: always the library GEMM); ``linear_norm_rows`` (default 32): up to that
many rows the residual norms run as prologues of the projections behind them; ``fused_lm_head`` (default true): LM head and sampler as one pass
over the weights for at most 64 rows (``lm_head_sample``), otherwise the library GEMM and ``sample_tokens``.
"""
from __future__ import annotations

import time

import torch

from minivllm_amd.engine.metadata import decode_metadata, prefill_metadata
from minivllm_amd.layers.attention import decode_workspace_bytes
from minivllm_amd.layers.basic import Sampler
from minivllm_amd.layers.fused import (decode_advance, lm_head_sample, lm_head_sample_takes,
                                       lm_head_sample_workspace_bytes, sample_tokens, sample_tokens_into,
                                       sample_workspace_bytes)
from minivllm_amd.models.qwen3 import Qwen3ForCausalLM
from minivllm_amd.utils.context import get_context, reset_context, set_context

_DTYPES = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16, "fp16": torch.float16, "float16": torch.float16,
           "fp32": torch.float32, "float32": torch.float32}


class PendingTokens:
    """Token ids of a launched decode step on their way to the host: the step's last kernel writes them into a
    row of pinned memory and then the step's sequence number into the row's last entry.

    The row is polled while the kernel may still be running, which is only meaningful for coherent (fine-grained)
    pinned host memory, what torch's pinned allocations are on ROCm unless the process runs with
    HIP_HOST_COHERENT=0.  With non-coherent pinned memory a write becomes visible at a synchronisation point only,
    so the poll gives up after a few milliseconds and synchronises the launch stream: slower, never wrong."""

    SPIN_SECONDS = 2e-3          # a decode step takes tens of microseconds; past this the host stops burning a core

    def __init__(self, row, count: int, sequence: int, stream=None):
        self.row, self.count, self.sequence = row, count, sequence     # row: numpy view of the pinned row
        self.stream = stream

    def wait(self) -> list[int]:
        row, want = self.row, self.sequence
        if int(row[-1]) != want:
            give_up = time.monotonic() + self.SPIN_SECONDS
            polls = 0
            while int(row[-1]) != want:
                polls += 1
                if polls & 0x3ff == 0:
                    if time.monotonic() > give_up:
                        break
                    time.sleep(0)                          # let another thread of the process run
            if int(row[-1]) != want:
                # blocks without spinning, makes non-coherent pinned memory visible, surfaces a device error
                (self.stream.synchronize() if self.stream is not None else torch.cuda.synchronize())
                if int(row[-1]) != want:
                    raise RuntimeError("decode step finished without delivering its token ids")
        return row[:self.count].tolist()


class ModelRunner:
    def __init__(self, config: dict, device: str = "cuda:0"):
        self.config = config
        self.device = torch.device(device)
        self.block_size = config.get("block_size", 256)
        self.num_blocks = config.get("max_cached_blocks", 1024)
        self.dtype = _DTYPES[config.get("dtype", "bf16")]
        self.kv_cache_dtype = config.get("kv_cache_dtype", "auto")
        head_dim = config.get("head_dim") or config["hidden_size"] // config["num_heads"]
        self.model = Qwen3ForCausalLM(
            vocab_size=config["vocab_size"], hidden_size=config["hidden_size"], num_heads=config["num_heads"],
            head_dim=head_dim, scale=config.get("scale", 1.0), num_kv_heads=config.get("num_kv_heads"),
            rms_norm_epsilon=config.get("rms_norm_epsilon", 1e-6), qkv_bias=config.get("qkv_bias", False),
            base=config.get("base", 1_000_000), max_position=config.get("max_position", 4096),
            intermediate_size=config["intermediate_size"], ffn_bias=config.get("ffn_bias", True),
            num_layers=config["num_layers"], tie_word_embeddings=config.get("tie_word_embeddings", True),
            block_size=self.block_size, kv_cache_dtype=self.kv_cache_dtype,
            fused_qk=config.get("fused_qk", True), fused_elementwise=config.get("fused_elementwise", True),
            small_rows=config.get("linear_small_rows", 64), norm_rows=config.get("linear_norm_rows", 32))
        self.model.reset_parameters(seed=config.get("seed", 0))
        self.model.to(device=self.device, dtype=self.dtype).eval()
        self.sampler = Sampler()
        self.fused_sampler = config.get("fused_sampler", True)
        self.fused_lm_head = self.fused_sampler and config.get("fused_lm_head", True)
        self.seed = config.get("seed", 0)
        self.sample_calls = 0
        self._pinned = None          # (2, max batch) pinned ids, written by the captured step itself
        self._dev_step = None        # host mirror of the graphs' device-side sampler call counter
        self._steady = None          # description of the batch in the static decode buffers (graph decode)
        self._last_sampled = None    # device tensor of the ids sampled by the last graph decode step
        self.generator = torch.Generator(device=self.device).manual_seed(config.get("seed", 0))
        self.allocate_kv_cache()
        self.graphs = {}
        if not config.get("enforce_eager", True):
            self.capture_decode_graphs()

    def allocate_kv_cache(self):
        """One pool ``[2, L, num_blocks, block_size, Hkv, D]``; each ``Attention`` gets its layer's views
        (model_runner.py:140-168).  With an INT8 cache a second pool holds the fp32 scales."""
        cfg = self.config
        hkv = cfg.get("num_kv_heads") or cfg["num_heads"]
        d = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_heads"]
        layers = cfg["num_layers"]
        int8 = self.kv_cache_dtype == "int8"
        self.kv_cache = torch.zeros(2, layers, self.num_blocks, self.block_size, hkv, d,
                                    dtype=torch.int8 if int8 else self.dtype, device=self.device)
        self.kv_scale = (torch.zeros(2, layers, self.num_blocks, self.block_size, hkv, dtype=torch.float32,
                                     device=self.device) if int8 else None)
        layer_id = 0
        for module in self.model.modules():
            if hasattr(module, "k_cache") and hasattr(module, "v_cache"):
                module.k_cache = self.kv_cache[0, layer_id]
                module.v_cache = self.kv_cache[1, layer_id]
                if int8:
                    module.k_scale = self.kv_scale[0, layer_id]
                    module.v_scale = self.kv_scale[1, layer_id]
                layer_id += 1
        assert layer_id == layers

    def _to_device(self, values, dtype):
        return torch.tensor(values, dtype=dtype, pin_memory=True).to(self.device, non_blocking=True)

    def prepare_prefill(self, seqs):
        """Packed prompt tokens and their metadata (model_runner.py:180-227).  Tokens covered by prefix-cache hits
        are left out and read from the paged cache by the attention kernel (also from an int8 cache, for 16-bit
        models with head_dim 128 or 64 and blocks of a multiple of 16 tokens); with ``prefix_caching=False`` they are
        recomputed into the shared blocks instead."""
        head_dim = self.config.get("head_dim") or self.config["hidden_size"] // self.config["num_heads"]
        int8_ok = self.dtype != torch.float32 and head_dim in (64, 128) and self.block_size % 16 == 0
        reuse = (self.kv_cache_dtype != "int8" or int8_ok) and self.config.get("prefix_caching", True)
        md = prefill_metadata(seqs, self.block_size, reuse_cached_kv=reuse)
        positions = [p for seq in seqs for p in range(seq.num_cached_tokens if reuse else 0, len(seq))]
        tables = md["block_tables"]
        set_context(True,
                    cu_seqlens_q=self._to_device(md["cu_seqlens_q"], torch.int32),
                    cu_seqlens_k=self._to_device(md["cu_seqlens_k"], torch.int32),
                    max_seqlen_q=md["max_seqlen_q"], max_seqlen_k=md["max_seqlen_k"],
                    slot_mapping=self._to_device(md["slot_mapping"], torch.int64),
                    context_lens=None,
                    block_tables=None if tables is None else self._to_device(tables, torch.int32))
        return self._to_device(md["input_ids"], torch.int64), self._to_device(positions, torch.int64)

    def decode_buckets(self):
        """Batch sizes a decode step is captured at (model_runner.py:316-369 uses the same ladder)."""
        max_bs = self.config.get("max_num_sequences", 16)
        return sorted({b for b in [1, 2, 4, 8] + list(range(16, max_bs + 1, 16)) + [max_bs] if b <= max_bs})

    def prepare_decode(self, seqs):
        md = decode_metadata(seqs, self.block_size)
        context_lens, slots, tables, ids = md["context_lens"], md["slot_mapping"], md["block_tables"], md["input_ids"]
        if self.config.get("eager_decode_as_captured", False) and len(seqs) <= self.config.get("max_num_sequences", 16):
            # The shapes a captured step has: the batch padded to its bucket with rows that store nothing and attend
            # to nothing, the block tables as wide as the longest sequence the model allows.  Every kernel then runs
            # on the plan (tiles, partitions) of the graph path, so an eager run reproduces a graph run bit for bit.
            cfg = self.config
            bucket = next(b for b in self.decode_buckets() if b >= len(seqs))
            max_len = cfg.get("max_model_length", cfg.get("max_position", 4096))
            width = -(-max_len // self.block_size)
            pad = bucket - len(seqs)
            tables = [list(t) + [0] * (width - len(t)) for t in tables] + [[0] * width] * pad
            context_lens = list(context_lens) + [0] * pad
            slots = list(slots) + [-1] * pad
            ids = list(ids) + [0] * pad
        context_lens = self._to_device(context_lens, torch.int64)
        set_context(False,
                    slot_mapping=self._to_device(slots, torch.int64),
                    context_lens=context_lens,
                    block_tables=self._to_device(tables, torch.int32))
        return self._to_device(ids, torch.int64), (context_lens - 1).clamp_(min=0)

    @torch.no_grad()
    def capture_decode_graphs(self):
        """Record one hipGraph of a whole decode step per batch-size bucket (model_runner.py:316-369): the forward
        pass, the LM head and the sampler.  Captured under ``no_grad``, not ``inference_mode`` (which the reference's
        capture runs under): torch creates the default generator's graph-side seed and offset tensors at the first
        capture and updates them in place at every later one, so captured in inference mode they would make every
        capture elsewhere in the process fail ("inplace update to inference tensor") for as long as these graphs live.

        The step metadata lives in static device buffers that ``run`` refills or advances before every replay;
        rows past the real batch carry slot -1, context length 0, temperature 1 and whatever table entries were
        there, which the kernels treat as "store nothing, output zeros".  The attention library allocates nothing
        and its grids depend only on the static shapes (batch bucket, table width), so a replay is valid for any
        contents of the buffers.  The sampler's call offset is a device counter that the graph itself increments
        (a replay cannot change a launch argument), kept equal to ``sample_calls``, so a run draws the same noise
        whether its steps are replayed or launched one by one."""
        cfg = self.config
        max_bs = cfg.get("max_num_sequences", 16)
        max_len = cfg.get("max_model_length", cfg.get("max_position", 4096))
        max_blocks = -(-max_len // self.block_size)
        dev = self.device
        buckets = self.decode_buckets()
        ws_bytes = max(sample_workspace_bytes(b, cfg["vocab_size"]) for b in buckets) if self.fused_sampler else 0
        lm_bytes = max(lm_head_sample_workspace_bytes(b, cfg["hidden_size"]) for b in buckets) if self.fused_lm_head else 0
        self.graph_vars = dict(
            input_ids=torch.zeros(max_bs, dtype=torch.int64, device=dev),
            positions=torch.zeros(max_bs, dtype=torch.int64, device=dev),
            slot_mapping=torch.full((max_bs,), -1, dtype=torch.int64, device=dev),
            context_lens=torch.zeros(max_bs, dtype=torch.int64, device=dev),
            block_tables=torch.zeros(max_bs, max_blocks, dtype=torch.int32, device=dev),
            temperatures=torch.ones(max_bs, dtype=torch.float32, device=dev),
            sampled=torch.zeros(max_bs, dtype=torch.int64, device=dev),
            step=torch.zeros(1, dtype=torch.int64, device=dev),
            sample_ws=torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev),
            lm_ws=torch.empty(max(lm_bytes, 16), dtype=torch.uint8, device=dev),
            outputs=torch.zeros(max_bs, cfg["hidden_size"], dtype=self.dtype, device=dev))
        v = self.graph_vars
        # the ids of a step, written by the step's last kernel into pinned host memory: row (sampler counter & 1)
        self._pinned = torch.zeros(2, max_bs + 1, dtype=torch.int64, pin_memory=True)
        self._pinned_rows = self._pinned.numpy()       # the same memory, for polling without tensor overhead
        self._own_decode_workspace(buckets, max_blocks)
        pool = None
        for bs in reversed(buckets):
            set_context(False, slot_mapping=v["slot_mapping"][:bs], context_lens=v["context_lens"][:bs],
                        block_tables=v["block_tables"][:bs])

            def forward():
                hidden = self.model(v["input_ids"][:bs], v["positions"][:bs])
                if not self.fused_sampler:                 # the module-chain sampler draws from a host-side generator
                    v["outputs"][:bs] = hidden
                    return
                if self.fused_lm_head and lm_head_sample_takes(hidden, self.model.lm_head_weight):
                    # LM head and sampler in one pass over the weights: no (bs, vocab) logits
                    lm_head_sample(hidden, self.model.lm_head_weight, v["temperatures"][:bs], self.seed, 0,
                                   out=v["sampled"][:bs], offset_dev=v["step"], workspace=v["lm_ws"])
                else:
                    logits = torch.nn.functional.linear(hidden, self.model.lm_head_weight)
                    nbytes = sample_workspace_bytes(bs, cfg["vocab_size"])
                    sample_tokens_into(v["sampled"][:bs], logits, v["temperatures"][:bs], self.seed, v["step"],
                                       v["sample_ws"][:nbytes] if nbytes else None)
                # the step ends with the next step's inputs (rows of padding stay) and the sampler's counter + 1:
                # a batch that goes on as it is needs nothing from the host but the rows that open a new block
                decode_advance(v["input_ids"][:bs], v["context_lens"][:bs], v["positions"][:bs],
                               v["slot_mapping"][:bs], v["sampled"][:bs], step=v["step"], host_ids=self._pinned)

            forward()                                    # warm-up outside the capture (library handles, lazy loads)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool):
                forward()
            pool = graph.pool() if pool is None else pool
            self.graphs[bs] = graph
            torch.cuda.synchronize()
            reset_context()
        self._dev_step = None                            # value of the device counter, unknown after the warm-ups
        torch.cuda.synchronize()
        self._pinned.zero_()                             # the warm-ups left their sequence numbers: steps count from 1

    def _own_decode_workspace(self, buckets, max_blocks):
        """One split-K scratch buffer for every decode call of this runner, allocated before any graph is
        captured and sized for the largest need over the batch buckets.  The need is not monotonic in the batch
        (a smaller batch is cut into more partitions), so a buffer grown bucket by bucket would be replaced,
        and freed, after a graph that holds its address had been captured."""
        cfg = self.config
        head_dim = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_heads"]
        need = max(decode_workspace_bytes(b, cfg["num_heads"], head_dim, max_blocks, self.block_size) for b in buckets)
        self.decode_workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=self.device)
        for module in self.model.modules():
            if hasattr(module, "decode_workspace"):
                module.decode_workspace = self.decode_workspace

    def _fill_decode_buffers(self, seqs, gbs):
        """Full refill of the static decode buffers from the host-side metadata (model_runner.py:231-256)."""
        bs = len(seqs)
        md = decode_metadata(seqs, self.block_size)
        v = self.graph_vars
        v["input_ids"][:bs].copy_(self._to_device(md["input_ids"], torch.int64))
        v["positions"][:gbs].zero_()
        v["positions"][:bs].copy_(self._to_device([n - 1 for n in md["context_lens"]], torch.int64))
        v["temperatures"][:gbs].fill_(1.0)
        v["temperatures"][:bs].copy_(self._to_device([seq.temperature for seq in seqs], torch.float32))
        v["slot_mapping"][:gbs].fill_(-1)
        v["slot_mapping"][:bs].copy_(self._to_device(md["slot_mapping"], torch.int64))
        v["context_lens"][:gbs].zero_()
        v["context_lens"][:bs].copy_(self._to_device(md["context_lens"], torch.int64))
        tables = self._to_device(md["block_tables"], torch.int32)
        v["block_tables"][:bs, :tables.size(1)].copy_(tables)
        self._steady = dict(key=tuple(seq.seq_id for seq in seqs), lens=[len(seq) for seq in seqs])

    def continues_last_decode(self, seqs) -> bool:
        """The same sequences as in the last graph decode step, each one token longer."""
        st = self._steady
        if st is None or self._last_sampled is None or st["key"] != tuple(seq.seq_id for seq in seqs):
            return False
        return all(len(seq) == m + 1 for seq, m in zip(seqs, st["lens"]))

    def _advance_decode_buffers(self, seqs) -> bool:
        """The same sequences as in the last graph decode step, each one token longer: the buffers were moved on by
        that step itself, on the device (input = the ids it sampled, context length and slot + 1), and only
        sequences that started a new block are patched from the host.  Returns False when the batch is not such a
        continuation."""
        if not self.continues_last_decode(seqs):
            return False
        st = self._steady
        lens = [len(seq) for seq in seqs]
        bs = len(seqs)
        v = self.graph_vars
        # the captured step has already moved its buffers on (decode_advance is its last launch)
        fresh = [i for i, n in enumerate(lens) if (n - 1) % self.block_size == 0]     # token n-1 opens a block
        if fresh:
            rows = self._to_device(fresh, torch.int64)
            cols = self._to_device([len(seqs[i].block_table) - 1 for i in fresh], torch.int64)
            blocks = [seqs[i].block_table[-1] for i in fresh]
            v["block_tables"][rows, cols] = self._to_device(blocks, torch.int32)
            v["slot_mapping"][rows] = self._to_device([b * self.block_size for b in blocks], torch.int64)
        st["lens"] = lens
        return True

    def _replay_decode(self, seqs):
        """One decode step from the captured graph; returns the sampled ids (a view of a static device buffer that
        the next replay overwrites), or with the module-chain sampler the hidden states."""
        bs = len(seqs)
        gbs = next(b for b in sorted(self.graphs) if b >= bs)
        if not self._advance_decode_buffers(seqs):
            self._fill_decode_buffers(seqs, gbs)
        v = self.graph_vars
        if self.fused_sampler and self._dev_step != self.sample_calls:
            v["step"].fill_(self.sample_calls)
        self.graphs[gbs].replay()
        if not self.fused_sampler:
            return v["outputs"][:bs]
        self.sample_calls += 1
        self._dev_step = self.sample_calls
        return v["sampled"][:bs]

    def can_launch_decode(self, seqs) -> bool:
        """A decode step of these sequences can be launched without waiting for its token ids: the captured graph
        covers the batch and the sampler is the single-launch one."""
        return bool(self.graphs) and len(seqs) <= max(self.graphs) and self.fused_sampler

    @torch.inference_mode()
    def launch_decode(self, seqs) -> "PendingTokens":
        """Enqueue one decode step and return at once; the step's last kernel writes the sampled ids into pinned host
        memory, followed by the step's sequence number (no copy operation and no event between two replays), and
        they are read with ``PendingTokens.wait()``.  The next step's input ids are taken from the device
        copy, so the host can schedule and launch step t + 1 while the GPU still runs step t.  When the batch
        does not continue the last step's, the buffers are refilled from the sequences' last tokens, which must be
        real by then (the caller commits outstanding ids first)."""
        calls = self.sample_calls                     # the counter's value when the step starts picks the pinned row
        sampled = self._replay_decode(seqs)
        self._last_sampled = sampled
        # step t's row is read after step t + 1 has been launched (into the other row)
        return PendingTokens(self._pinned_rows[calls & 1], len(seqs), calls + 1, torch.cuda.current_stream(self.device))

    @torch.inference_mode()
    def run(self, seqs, is_prefill: bool) -> list[int]:
        if not is_prefill and self.graphs and len(seqs) <= max(self.graphs):
            out = self._replay_decode(seqs)
            if self.fused_sampler:
                self._last_sampled = out                       # next step's input ids, if it continues this batch
                token_ids = out.tolist()
                reset_context()
                return token_ids
            logits = torch.nn.functional.linear(out, self.model.lm_head_weight)
            temperatures = self._to_device([seq.temperature for seq in seqs], torch.float32)
        else:
            input_ids, positions = self.prepare_prefill(seqs) if is_prefill else self.prepare_decode(seqs)
            rows_out = len(seqs) if is_prefill else input_ids.shape[0]     # decode: the padded batch, if padded
            temperatures = self._to_device([seq.temperature for seq in seqs] + [1.0] * (rows_out - len(seqs)), torch.float32)
            hidden = self.model(input_ids, positions)
            if (self.fused_sampler and self.fused_lm_head
                    and lm_head_sample_takes(hidden, self.model.lm_head_weight, rows_out)):
                # the rows to sample from are picked inside the kernel: the last token of every packed sequence in
                # prefill (embedding_head.py:57-62), every row in decode
                rows = (get_context().cu_seqlens_q[1:] - 1).long() if is_prefill else None
                sampled = lm_head_sample(hidden, self.model.lm_head_weight, temperatures, self.seed,
                                         self.sample_calls, row_index=rows)
                self.sample_calls += 1
                self._last_sampled = None
                self._steady = None
                token_ids = sampled.tolist()[:len(seqs)]
                reset_context()
                return token_ids
            logits = self.model.compute_logits(hidden)
        if self.fused_sampler:
            # one launch over the LM-head output; draws are a function of (seed, step), so a run is reproducible
            sampled = sample_tokens(logits, temperatures, self.seed, self.sample_calls)
            self.sample_calls += 1
        else:
            sampled = self.sampler(logits, temperatures, self.generator)
        self._last_sampled = None
        self._steady = None
        token_ids = sampled.tolist()[:len(seqs)]
        reset_context()
        return token_ids
