"""Host-side operator surface: Context record and argument checks (CPU only)."""
import pytest
import torch

from minivllm_amd.layers.attention import Attention, paged_attention_decode, store_kvcache
from minivllm_amd.utils import get_context, reset_context, set_context
from minivllm_amd._C import MinivllmAmdError


def test_context_positional_order_and_reset():
    t = torch.zeros(3, dtype=torch.int32)
    set_context(True, t, t, 7, 9, None, None, None)
    c = get_context()
    assert c.is_prefill and c.cu_seqlens_q is t and c.max_seqlen_q == 7 and c.max_seqlen_k == 9
    first = c
    set_context(False, slot_mapping=t, context_lens=t, block_tables=t)
    assert get_context() is not first and get_context().slot_mapping is t and not get_context().is_prefill
    reset_context()
    c = get_context()
    assert (c.is_prefill, c.cu_seqlens_q, c.slot_mapping, c.block_tables, c.max_seqlen_q) == (False, None, None, None, 0)


def test_attention_defaults_match_reference_constructor():
    a = Attention(num_heads=8, head_dim=64)
    assert a.num_kv_heads == 8 and a.block_size == 16 and a.scale == 1.0
    assert a.k_cache.numel() == 0 and a.v_cache.numel() == 0
    b = Attention(16, 128, 1.0, 8, 256)
    assert (b.num_heads, b.head_dim, b.num_kv_heads, b.block_size) == (16, 128, 8, 256)


def test_no_cpu_fallback():
    k = torch.zeros(4, 2, 8)
    cache = torch.zeros(2, 4, 2, 8)
    with pytest.raises(MinivllmAmdError):
        store_kvcache(k, k, cache, cache.clone(), torch.arange(4), 4)
    with pytest.raises(MinivllmAmdError):
        paged_attention_decode(torch.zeros(1, 4, 8), cache, cache, torch.zeros(1, 2, dtype=torch.int32),
                               torch.ones(1, dtype=torch.int32), 1.0, 4, 2, 8, 4)


def test_store_asserts_like_reference():
    k = torch.zeros(4, 2, 8)
    with pytest.raises(AssertionError):
        store_kvcache(k, k, torch.zeros(2, 4, 2, 8), torch.zeros(3, 4, 2, 8), torch.arange(4), 4)
    with pytest.raises(AssertionError):
        store_kvcache(k, k, torch.zeros(2, 4, 2, 8), torch.zeros(2, 4, 2, 8), torch.arange(3), 4)


def test_prefill_without_cu_seqlens_raises_value_error():
    set_context(True)
    a = Attention(4, 8, 1.0, 2, 4)
    with pytest.raises(ValueError):
        a(torch.zeros(3, 4, 8), torch.zeros(3, 2, 8), torch.zeros(3, 2, 8))
    with pytest.raises(ValueError):                    # neither packed (3-D) nor batched (4-D)
        a(torch.zeros(1, 1, 3, 4, 8), torch.zeros(1, 1, 3, 2, 8), torch.zeros(1, 1, 3, 2, 8))
    from minivllm_amd._C import MinivllmAmdError
    with pytest.raises(MinivllmAmdError):              # batched 4-D prefill is the packed kernel: no CPU path
        a(torch.zeros(1, 3, 4, 8), torch.zeros(1, 3, 2, 8), torch.zeros(1, 3, 2, 8))
    reset_context()


def test_bench_refuses_more_than_one_gpu_and_a_machine_without_one():
    """bench.py measures one GPU: --gpus above 1 exits with a message; without a GPU it says so instead of
    timing anything else (there is no CPU path to fall back to)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)
    import torch
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "1", "--warmup", "0"],
                           capture_output=True, text=True)
        assert r.returncode != 0 and "no GPU" in (r.stdout + r.stderr)
