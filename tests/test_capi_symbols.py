"""The C-ABI library loads and exports every symbol include/minivllm_amd.h declares.
No compute calls: there is no GPU here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "minivllm_amd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mvllm_[a-z0-9_]+)\s*\(", text)))


def _lib():
    from minivllm_amd import _C
    if not os.path.exists(_C.lib_path()):
        from minivllm_amd._build import build_library
        build_library(verbose=False)
    return _C


def test_header_declares_expected_entry_points():
    names = _declared()
    for n in ["mvllm_store_kvcache", "mvllm_store_kvcache_int8", "mvllm_paged_decode",
              "mvllm_paged_decode_int8", "mvllm_paged_decode_noalloc", "mvllm_paged_decode_workspace_bytes", "mvllm_paged_decode_plan", "mvllm_prefill_plan", "mvllm_prefill_varlen",
              "mvllm_prefill_paged", "mvllm_prefill_paged_int8", "mvllm_prefill_paged_int8_staged", "mvllm_prefill_paged_staged", "mvllm_prefill_paged_staged_workspace_bytes", "mvllm_prefill_paged_split", "mvllm_prefill_paged_int8_split", "mvllm_prefill_paged_split_plan", "mvllm_prefill_paged_split_workspace_bytes", "mvllm_qk_norm_rope_store", "mvllm_sample_tokens", "mvllm_sample_tokens_dev_offset", "mvllm_decode_advance", "mvllm_sample_tokens_workspace_bytes",
              "mvllm_add_rms_norm", "mvllm_linear_small_m", "mvllm_norm_linear_small_m", "mvllm_linear_small_m_plan",
              "mvllm_lm_head_sample", "mvllm_lm_head_sample_workspace_bytes",
              "mvllm_silu_and_mul", "mvllm_version", "mvllm_status_string"]:
        assert n in names


def test_library_exports_every_declared_symbol():
    _C = _lib()
    raw = ctypes.CDLL(_C.lib_path())
    for name in _declared():
        assert hasattr(raw, name), f"{name} declared in the header but not exported"
    assert set(_C.SIGNATURES) == set(_declared())


def test_host_only_entry_points():
    _C = _lib()
    lib = _C.load()
    assert lib.mvllm_version() >= 1000
    assert lib.mvllm_status_string(-5).decode().startswith("workspace")
    # pure host arithmetic: (D + 2) floats per (seq, partition, head); partitions of 256..1024 tokens, at most 32
    # per sequence, shortened down to 64 tokens while batch * partitions < 1024
    assert lib.mvllm_paged_decode_workspace_bytes(1024, 16, 128, 16, 16) == 0        # 256 tokens: 1 partition
    assert lib.mvllm_paged_decode_workspace_bytes(8, 16, 128, 16, 16) == 8 * 4 * 16 * 130 * 4     # 4 x 64 tokens
    assert lib.mvllm_paged_decode_workspace_bytes(2, 4, 128, 64, 16) == 2 * 16 * 4 * 130 * 4      # 16 x 64 tokens
    assert lib.mvllm_paged_decode_workspace_bytes(256, 32, 128, 2048, 16) == 256 * 32 * 32 * 130 * 4


def test_prefill_split_plan_is_host_arithmetic():
    """When a paged prefill is cut over its keys: few query tiles, at least 4096 keys, a shape the split form takes;
    and the workspace holds the ranges' tables, partial results and denominators."""
    _C = _lib()
    lib = _C.load()
    bf16, f32 = 1, 0
    plan = lib.mvllm_prefill_paged_split_plan
    assert plan(1, 128, 32768 + 128, 32, 8, 128, 256, bf16, 0) == 16          # 32 workgroups a range: 15 prefix ranges
    assert plan(1, 16, 32768 + 16, 32, 8, 128, 256, bf16, 0) == 17            # never more than 16 prefix ranges
    assert plan(2, 256, 4096 + 128, 32, 8, 128, 16, bf16, 0) == 5             # 1024 keys a range at least
    assert plan(2, 1024, 16384 + 512, 32, 8, 128, 256, bf16, 0) == 5          # a small batch is cut in 4 at least
    assert plan(16, 512, 4096 + 32, 32, 8, 128, 256, bf16, 0) == 0            # enough query tiles
    assert plan(1, 128, 4095, 32, 8, 128, 256, bf16, 0) == 0                  # too few keys
    assert plan(1, 128, 32768, 32, 8, 128, 256, f32, 0) == 0                  # fp32
    assert plan(1, 128, 32768, 32, 8, 128, 8, bf16, 0) == 0                   # blocks of 8 tokens
    assert plan(1, 128, 32768 + 128, 32, 8, 128, 256, bf16, 1) == 16          # INT8 cache: as the 16-bit one
    assert plan(1, 128, 32768, 32, 8, 80, 256, bf16, 1) == 0                  # ... but at head_dim 64 / 128 only
    assert plan(1, 128, 32768, 16, 8, 80, 256, bf16, 0) == 17                 # head_dim 80: 16 workgroups a range
    assert plan(8, 4096, 32768, 16, 8, 80, 256, bf16, 0) == 0                 # ... 576 of them fill the chip
    assert plan(1, 128, 32768, 16, 8, 72, 256, bf16, 0) == 17                 # head_dim 72: as 80
    assert plan(1, 128, 32768, 16, 8, 136, 256, bf16, 0) == 0                 # head_dim 136: not an LDS-tiled shape
    need = lib.mvllm_prefill_paged_split_workspace_bytes(1, 128, 32768 + 128, 32, 8, 128, 256, bf16, 16)
    partial = 16 * 128 * 32 * 128 * 2 + 16 * 128 * 32 * 4
    assert partial < need < partial + 16384
    assert lib.mvllm_prefill_paged_split_workspace_bytes(8, 128, 32768, 32, 8, 128, 256, bf16, 9) == 0   # 72 ranges


def test_decode_plan_is_host_arithmetic():
    """Which form a decode call takes, and that the split form never needs more workspace than is advertised."""
    import torch
    from minivllm_amd.layers.attention import paged_decode_plan
    lib = _lib().load()
    # one-wave-per-head form: large batch over a wide table (1024-token partitions)
    assert paged_decode_plan(256, 32, 8, 128, 2048, 16) == (1024, 32, 1)
    assert paged_decode_plan(64, 32, 8, 128, 2048, 16) == (1024, 32, 1)
    # small-batch form: 64 sequences x 8 kv heads in a 4096-token table are one partition each, four waves per head
    assert paged_decode_plan(64, 32, 8, 128, 256, 16) == (4096, 1, 4)
    assert paged_decode_plan(256, 32, 8, 128, 16, 256) == (4096, 1, 4)        # any batch while the table is <= 4096
    assert paged_decode_plan(1, 32, 8, 128, 2048, 16) == (1024, 32, 4)        # one long sequence: 256 workgroups
    assert paged_decode_plan(16, 32, 8, 128, 512, 16) == (2048, 4, 4)
    # INT8 caches, and shapes outside the MFMA kernels
    assert paged_decode_plan(64, 32, 8, 128, 256, 16, int8_cache=True) == (4096, 1, 4)
    assert paged_decode_plan(256, 32, 8, 128, 256, 16, int8_cache=True) == (1024, 4, 1)     # large INT8 batch: first form
    assert paged_decode_plan(64, 16, 16, 64, 256, 16)[2] == 4                 # head_dim 64: MFMA kernels, both cache types
    assert paged_decode_plan(64, 16, 16, 64, 256, 16, int8_cache=True)[2] == 1      # 1024 (sequence, head) pairs: first form
    assert paged_decode_plan(64, 16, 16, 96, 256, 16, int8_cache=True)[2] == 0
    assert paged_decode_plan(64, 16, 16, 96, 256, 16)[2] == 4                 # 16-bit caches: also 96 dims (three 32-dim steps)
    assert paged_decode_plan(64, 16, 16, 80, 256, 16)[2] == 4 and paged_decode_plan(64, 16, 16, 112, 256, 16)[2] == 4   # ... and a partial last step
    assert paged_decode_plan(64, 16, 16, 72, 256, 16)[2] == 4 and paged_decode_plan(64, 16, 16, 120, 256, 16)[2] == 4   # any multiple of 8 from 32 to 128
    assert paged_decode_plan(64, 16, 16, 100, 256, 16)[2] == 0 and paged_decode_plan(64, 16, 16, 136, 256, 16)[2] == 0   # other head dims
    assert paged_decode_plan(64, 16, 16, 72, 256, 16, dtype=torch.float32)[2] == 0
    assert paged_decode_plan(64, 16, 8, 256, 256, 16)[2] == 4                 # 16-bit caches: also 256 and 32 dims
    assert paged_decode_plan(64, 16, 8, 32, 256, 16)[2] == 4
    assert paged_decode_plan(64, 16, 8, 256, 256, 16, int8_cache=True)[2] == 0
    assert paged_decode_plan(64, 16, 8, 256, 256, 16, dtype=__import__("torch").float32)[2] == 0
    assert paged_decode_plan(64, 32, 8, 128, 256, 16, dtype=torch.float32)[2] == 4       # fp32 caches: fp32 MFMA
    assert paged_decode_plan(64, 32, 8, 128, 256, 16, dtype=torch.float32, int8_cache=True)[2] == 0
    assert paged_decode_plan(8, 34, 2, 128, 64, 16)[2] == 4                   # 17 query heads per kv head: two slices each
    # the advertised workspace covers whatever form is chosen
    for batch in (1, 3, 16, 64, 200, 1000):
        for blocks, bs in ((16, 16), (64, 16), (300, 16), (2048, 16), (40, 256), (70000, 16)):
            for hkv in (1, 2, 8):
                part, parts, waves = paged_decode_plan(batch, 8 * hkv, hkv, 128, blocks, bs)
                assert part % 16 == 0 and parts == -(-blocks * bs // part) and 1 <= parts <= 32
                need = 0 if parts == 1 else batch * parts * 8 * hkv * 130 * 4
                assert need <= lib.mvllm_paged_decode_workspace_bytes(batch, 8 * hkv, 128, blocks, bs)


def test_prefill_plan_is_host_arithmetic():
    """Which kernel a prefill takes: 2 LDS-tiled MFMA, 1 16-row tile MFMA, 0 generic."""
    import torch
    from minivllm_amd.layers.attention import prefill_plan
    assert prefill_plan(32, 8, 128) == 2 and prefill_plan(16, 8, 64, dtype=torch.float16) == 2
    assert prefill_plan(32, 8, 128, block_size=16) == 2 and prefill_plan(32, 8, 128, block_size=8) == 0
    assert prefill_plan(32, 8, 128, dtype=torch.float32) == 2 and prefill_plan(16, 8, 64, 16, torch.float32) == 2     # fp32: its own LDS-tiled kernel
    assert prefill_plan(16, 8, 64, 8, torch.float32) == 0
    assert prefill_plan(8, 8, 256) == 2 and prefill_plan(8, 8, 32, block_size=32) == 2      # bf16 / fp16 only
    assert prefill_plan(8, 8, 256, dtype=torch.float32) == 0
    assert prefill_plan(6, 2, 80) == 2 and prefill_plan(6, 2, 96) == 2 and prefill_plan(6, 2, 96, dtype=torch.float32) == 0
    assert prefill_plan(6, 2, 112, block_size=16) == 2 and prefill_plan(6, 2, 112, block_size=8) == 0
    assert prefill_plan(6, 2, 72) == 2 and prefill_plan(6, 2, 40) == 2 and prefill_plan(6, 2, 48) == 2 and prefill_plan(6, 2, 100) == 0
    assert prefill_plan(6, 2, 120, block_size=32) == 2 and prefill_plan(6, 2, 72, dtype=torch.float32) == 0
    assert prefill_plan(6, 2, 136) == 0 and prefill_plan(6, 2, 24) == 0
    assert prefill_plan(32, 8, 128, 16, int8_cache=True) == 2
    assert prefill_plan(32, 8, 96, 16, int8_cache=True) == -1 and prefill_plan(32, 8, 128, 16, torch.float32, True) == -1
    assert prefill_plan(8, 8, 1024) == -1


def test_generic_kernel_warning_is_raised_once_per_shape():
    import warnings
    import torch
    from minivllm_amd.layers import attention
    attention._shapes_seen.clear()
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        attention._warn_if_generic("decode", 16, 16, 100, 16, torch.bfloat16, False)
        attention._warn_if_generic("decode", 16, 16, 100, 16, torch.bfloat16, False)      # same shape: silent
        attention._warn_if_generic("prefill", 6, 2, 100, 0, torch.bfloat16, False)
        attention._warn_if_generic("decode", 32, 8, 128, 16, torch.bfloat16, False)      # MFMA kernel: silent
        attention._warn_if_generic("prefill", 32, 8, 128, 0, torch.bfloat16, False)
    assert len(seen) == 2 and all("generic kernel" in str(w.message) for w in seen)


def test_argument_validation_without_gpu():
    """Invalid arguments are rejected before any launch, so this is safe on CPU."""
    _C = _lib()
    lib = _C.load()
    assert lib.mvllm_store_kvcache(0, 0, 0, 0, 0, 4, 16, 2, 8, 7, 0) == -2      # bad dtype
    assert lib.mvllm_store_kvcache(0, 0, 0, 0, 0, 4, 16, 0, 8, 1, 0) == -3      # bad shape
    assert lib.mvllm_store_kvcache(0, 0, 0, 0, 0, 4, 16, 2, 8, 1, 0) == -1      # null pointers
    assert lib.mvllm_store_kvcache(0, 0, 0, 0, 0, 0, 16, 2, 8, 1, 0) == 0       # empty is a no-op
    assert lib.mvllm_store_kvcache_int8(0, 0, 0, 0, 0, 0, 0, 4, 16, 2, 12, 1, 0) == -4   # D % 8 != 0
    assert lib.mvllm_paged_decode(0, 0, 0, 0, 0, 4, 0, 1, 2, 6, 4, 128, 16, 8, 1.0, 1, 0, 0, 0) == -3  # Hq % Hkv
    noalloc = lib.mvllm_paged_decode_noalloc
    assert noalloc(0, 0, 0, 0, 0, 4, 0, 1, 2, 6, 4, 128, 16, 8, 1.0, 1, 0) == -3                       # Hq % Hkv
    assert noalloc(1, 1, 1, 1, 1, 2048, 1, 1, 256, 32, 8, 128, 16, 8, 1.0, 1, 0) == -5                 # beyond the static array: refused before any launch
    assert lib.mvllm_prefill_varlen(0, 0, 0, 0, 0, 0, 0, 4, 2, 128, 1.0, 1, 0) == 0      # empty batch
    assert lib.mvllm_prefill_varlen(0, 0, 0, 0, 0, 1, 5, 4, 2, 128, 1.0, 1, 0) == -1
    paged = lib.mvllm_prefill_paged
    #            out q kc vc tables MB cu_q cu_k S  T  Hq Hkv D   bs  NB scale dt stream
    assert paged(0, 0, 0, 0, 0, 4, 0, 0, 0, 0, 4, 2, 128, 16, 8, 1.0, 1, 0) == 0       # no sequences
    assert paged(0, 0, 0, 0, 0, 4, 0, 0, 1, 5, 4, 2, 128, 16, 8, 1.0, 1, 0) == -1      # null pointers
    assert paged(0, 0, 0, 0, 0, 4, 0, 0, 1, 5, 4, 3, 128, 16, 8, 1.0, 1, 0) == -3      # Hq % Hkv
    assert paged(0, 0, 0, 0, 0, 4, 0, 0, 1, 5, 4, 2, 128, 0, 8, 1.0, 1, 0) == -3       # block_size
    sample = lib.mvllm_sample_tokens
    assert sample(0, 0, 100, 0, 0, 1, 2, 0, 100, 1, 0, 0, 0) == 0        # empty batch
    assert sample(0, 0, 100, 0, 0, 1, 2, 4, 100, 1, 0, 0, 0) == -1       # null pointers
    assert sample(0, 0, 50, 0, 0, 1, 2, 4, 100, 1, 0, 0, 0) == -3        # row stride < vocab
    assert sample(0, 0, 100, 0, 0, 1, 2, 4, 100, 5, 0, 0, 0) == -2       # dtype
    ws = lib.mvllm_sample_tokens_workspace_bytes
    assert ws(64, 151936) == 64 * 8 * 8 and ws(1024, 151936) == 0 and ws(4, 1000) == 0 and ws(1, 151936) == 38 * 8
    norm = lib.mvllm_add_rms_norm
    assert norm(0, 0, 0, 0, 0, 1e-6, 0, 1024, 1024, 1024, 1, 0) == 0       # no rows
    assert norm(0, 0, 0, 0, 0, 1e-6, 4, 1024, 1024, 1024, 1, 0) == -1      # null pointers
    assert norm(0, 0, 0, 0, 0, 1e-6, 4, 1004, 1004, 1004, 1, 0) == -4      # hidden % 8
    assert norm(0, 0, 0, 0, 0, 1e-6, 4, 1024, 512, 1024, 1, 0) == -3       # stride < hidden
    act = lib.mvllm_silu_and_mul
    assert act(0, 0, 0, 3072, 6144, 1, 0) == 0
    assert act(0, 0, 2, 3072, 6144, 1, 0) == -1
    assert act(0, 0, 2, 3072, 3072, 1, 0) == -3                            # stride < 2 * width
    assert act(0, 0, 2, 3001, 6002, 1, 0) == -4                            # width not a multiple of 16 bytes
    lin = lib.mvllm_linear_small_m
    assert lin(0, 0, 0, 0, 1024, 0, 4096, 1024, 1, 0) == 0                 # no rows
    assert lin(0, 0, 0, 0, 1024, 4, 4096, 1024, 1, 0) == -1                # null pointers
    assert lin(16, 16, 16, 0, 1024, 65, 4096, 1024, 1, 0) == -4            # more than 64 rows: the library GEMM's
    assert lin(16, 16, 16, 0, 1024, 4, 4100, 1024, 1, 0) == -4             # N % 16
    assert lin(16, 16, 16, 0, 1000, 4, 4096, 1000, 1, 0) == -4             # K % 512
    assert lin(16, 16, 16, 0, 512, 4, 4096, 1024, 1, 0) == -3              # row stride < K
    assert lin(16, 16, 16, 0, 1024, 4, 4096, 1024, 0, 0) == -4             # fp32
    nl = lib.mvllm_norm_linear_small_m
    #    out res_out x res gamma eps w bias stride M N K glu dtype stream
    assert nl(0, 0, 0, 0, 0, 1e-6, 0, 0, 1024, 0, 4096, 1024, 0, 1, 0) == 0          # no rows
    assert nl(0, 0, 0, 0, 0, 1e-6, 0, 0, 1024, 4, 4096, 1024, 0, 1, 0) == -1         # null pointers
    assert nl(16, 0, 16, 16, 0, 1e-6, 16, 0, 1024, 4, 4096, 1024, 0, 1, 0) == -1     # a residual without gamma
    assert nl(16, 32, 32, 48, 64, 1e-6, 16, 0, 1024, 4, 4096, 1024, 0, 1, 0) == -3   # residual_out aliases x
    assert nl(16, 0, 16, 0, 0, 1e-6, 16, 0, 1024, 4, 4112, 1024, 1, 1, 0) == -4      # glu: N % 32
    plan = lib.mvllm_linear_small_m_plan
    w = ctypes.c_int(0)
    assert plan(16, 4096, 1024, 1, 0, 1, ctypes.byref(w)) == 0 and w.value == 4     # the engine's QKV projection
    assert plan(32, 6144, 1024, 1, 1, 1, ctypes.byref(w)) == 0 and w.value == 4     # gate/up with norm and SiLU
    assert plan(33, 4096, 1024, 1, 0, 1, ctypes.byref(w)) == 0 and w.value == 4     # 17 rows and more: a workgroup per 16 rows
    assert plan(64, 6144, 1024, 1, 1, 1, ctypes.byref(w)) == 0 and w.value == 4
    assert plan(33, 4096, 1024, 0, 0, 1, None) == 0                                 # plain: up to 64
    assert plan(16, 1024, 3072, 1, 0, 1, None) == -4                                # K / waves is not one burst
    assert plan(16, 1024, 2048, 1, 0, 1, ctypes.byref(w)) == 0 and w.value == 16    # 16 waves, 128 values each
    assert plan(32, 1024, 2048, 1, 0, 1, ctypes.byref(w)) == 0 and w.value == 8     # two row tiles: twice the workgroups, half the waves
    assert plan(16, 4096, 1024, 1, 0, 0, None) == -4 and plan(16, 4096, 1024, 1, 0, 9, None) == -2
    lm = lib.mvllm_lm_head_sample
    #   out hidden stride row_index weight temps seed offset offset_dev batch vocab K dtype ws ws_bytes stream
    assert lm(0, 0, 1024, 0, 0, 0, 0, 0, 0, 0, 151936, 1024, 1, 0, 0, 0) == 0                  # no rows
    assert lm(0, 0, 1024, 0, 0, 0, 0, 0, 0, 4, 151936, 1024, 1, 0, 0, 0) == -1                 # null pointers
    assert lm(8, 16, 1024, 0, 16, 8, 0, 0, 0, 65, 151936, 1024, 1, 0, 0, 0) == -4              # more than 64 rows
    assert lm(8, 16, 1024, 0, 16, 8, 0, 0, 0, 4, 151930, 1024, 1, 0, 0, 0) == -4               # vocab % 16
    assert lm(8, 16, 768, 0, 16, 8, 0, 0, 0, 4, 151936, 768, 1, 0, 0, 0) == -4                 # hidden size
    assert lm(8, 16, 1024, 0, 16, 8, 0, 0, 0, 4, 151936, 1024, 0, 0, 0, 0) == -4               # fp32
    assert lm(8, 16, 1024, 0, 16, 8, 0, 0, 0, 4, 151936, 1024, 1, 0, 0, 0) == -5               # no workspace
    wsb = lib.mvllm_lm_head_sample_workspace_bytes
    assert wsb(16, 1024) == 16 * 512 * 8 and wsb(64, 1024) == 64 * 256 * 8 and wsb(65, 1024) == 0
    adv = lib.mvllm_decode_advance
    assert adv(0, 0, 0, 0, 0, 0, 0, 0, 0, 0) == 0 and adv(0, 0, 0, 0, 0, 0, 0, 0, 4, 0) == -1
    assert adv(0, 0, 0, 0, 0, 0, 0, 0, -1, 0) == -3 and adv(8, 8, 8, 8, 8, 0, 8, 8, 4, 0) == -1     # host ids without the counter
    assert adv(8, 8, 8, 8, 8, 8, 8, 4, 4, 0) == -3                                                # host rows shorter than the batch + 1
    assert lib.mvllm_sample_tokens_dev_offset(8, 8, 100, 8, 1, 0, 4, 100, 1, 0, 0, 0) == -1       # no counter
    fused = lib.mvllm_qk_norm_rope_store
    #     q_out k_out v_out q k v | strides | gamma eps cos max_pos pos slots | caches scales int8 | T slots Hq Hkv D dt stream
    assert fused(0, 0, 0, 0, 0, 0, 512, 256, 256, 0, 1e-6, 0, 64, 0, 0, 0, 0, 0, 0, 0, 0, 0, 4, 2, 128, 1, 0) == 0   # no tokens
    assert fused(0, 0, 0, 0, 0, 0, 512, 256, 256, 0, 1e-6, 0, 64, 0, 0, 0, 0, 0, 0, 0, 3, 0, 4, 2, 128, 1, 0) == -1  # nulls
    assert fused(0, 0, 0, 0, 0, 0, 512, 256, 256, 0, 1e-6, 0, 64, 0, 0, 0, 0, 0, 0, 0, 3, 0, 4, 2, 100, 1, 0) == -4  # D % 8
    assert fused(0, 0, 0, 0, 0, 0, 100, 256, 256, 0, 1e-6, 0, 64, 0, 0, 0, 0, 0, 0, 0, 3, 0, 4, 2, 128, 1, 0) == -3  # stride < row
    assert fused(0, 0, 0, 0, 0, 0, 512, 256, 256, 0, 1e-6, 0, 64, 0, 0, 0, 0, 0, 0, 0, 3, 0, 4, 2, 128, 9, 0) == -2  # dtype
    with pytest.raises(ValueError):
        _C.check(-3, "x")
    with pytest.raises(RuntimeError):
        _C.check(700, "x")
