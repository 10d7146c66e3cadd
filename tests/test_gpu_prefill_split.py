"""Paged prefill with every sequence's keys cut into ranges (mvllm_prefill_paged_split) against the CPU oracle and
against the one-step form."""
import math

import pytest
import torch

import oracle
from helpers import error_stats, make_paged_prefill_case
from minivllm_amd.layers.attention import flash_attention_prefill_paged

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16 = 2e-2, 2e-3


def _run(c, hq, hkv, d, bs, scale, splits, max_k):
    return flash_attention_prefill_paged(c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV),
                                         c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
                                         hq, hkv, d, bs, max_seqlen_k=max_k, key_splits=splits).cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached,splits", [
    (32, 8, 128, 16, [1300], [1200], 4),                           # one sequence, three prefix ranges and the tail
    (32, 8, 128, 16, [1300, 90, 700, 64], [1237, 0, 699, 63], 3),  # prefixes off the tile grid, none, one new token
    (16, 8, 128, 256, [2100, 800], [2000, 512], 5),                # the engine's block size: ranges of whole blocks
    (12, 2, 64, 48, [1000, 400, 30], [900, 200, 7], 6),            # ranges of 192 keys (blocks of 48), head_dim 64
    (5, 5, 128, 32, [600, 130], [500, 100], 2),                    # no grouping: one head per workgroup
    (32, 8, 128, 16, [200, 100], [100, 40], 8),                    # more ranges than the prefixes have tiles
    (8, 1, 64, 64, [3000], [2990], 16),                            # one kv head, ten new tokens
])
def test_paged_prefill_split_over_keys(hq, hkv, d, bs, lengths, cached, splits, dtype):
    c = make_paged_prefill_case(83, lengths, cached, hq, hkv, d, bs, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(c, hq, hkv, d, bs, scale, splits, max(lengths))
    assert not torch.isnan(got.float()).any()
    want = oracle.prefill_paged_oracle(c["q_new"].float(), torch.nan_to_num(c["k_cache"].float()),
                                       torch.nan_to_num(c["v_cache"].float()), c["block_tables"], c["cu_q"], c["cu_k"],
                                       scale, hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    one_step = _run(c, hq, hkv, d, bs, scale, 0, max(lengths))
    mx, mean = error_stats(got, one_step.float())
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


def test_paged_prefill_splits_by_itself_behind_a_long_prefix():
    """Without key_splits the library's plan decides: 40 new tokens behind 4200 cached ones are cut, and the result
    agrees with the oracle; the same call without the host's bound on the key count runs in one step."""
    hq, hkv, d, bs = 8, 2, 128, 16
    lengths, cached = [4240, 4100], [4200, 4090]
    from minivllm_amd import _C
    assert _C.load().mvllm_prefill_paged_split_plan(2, 50, 4240, hq, hkv, d, bs, _C.dtype_code(torch.bfloat16), 0) >= 3
    c = make_paged_prefill_case(89, lengths, cached, hq, hkv, d, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    got = _run(c, hq, hkv, d, bs, scale, None, max(lengths))
    want = oracle.prefill_paged_oracle(c["q_new"].float(), torch.nan_to_num(c["k_cache"].float()),
                                       torch.nan_to_num(c["v_cache"].float()), c["block_tables"], c["cu_q"], c["cu_k"],
                                       scale, hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    one_step = _run(c, hq, hkv, d, bs, scale, None, None)
    assert not torch.equal(one_step, got)                 # two different summation orders
    mx, mean = error_stats(one_step, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


def test_split_plan_and_rejections():
    from minivllm_amd import _C
    lib = _C.load()
    bf = _C.dtype_code(torch.bfloat16)
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 128, 256, bf, 0) >= 3
    assert lib.mvllm_prefill_paged_split_plan(16, 16384, 2048, 32, 8, 128, 256, bf, 0) == 0      # the chip is full
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 2048, 32, 8, 128, 256, bf, 0) == 0         # too few keys to cut
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 128, 256, bf, 1) == 0        # INT8 cache
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 80, 256, bf, 0) == 0         # head_dim 80
    assert lib.mvllm_prefill_paged_split_workspace_bytes(40, 128, 32768, 32, 8, 128, 256, bf, 2) == 0   # 80 ranges
    c = make_paged_prefill_case(5, [300], [200], 8, 8, 128, 16, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        _run(c, 8, 8, 128, 8, 0.1, 4, 300)                        # cache block dimension != block_size
