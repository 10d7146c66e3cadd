"""Paged prefill with every sequence's keys cut into ranges (mvllm_prefill_paged_split, mvllm_prefill_paged_int8_split)
against the CPU oracle and against the one-step form."""
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
    (16, 8, 80, 16, [900, 300], [800, 299], 4),                    # head_dim 80 in the layout of 128
    (6, 2, 32, 32, [700], [650], 3),                               # head_dim 32 in the layout of 64; three heads per kv head
    (8, 4, 256, 16, [600, 200], [520, 130], 3),                    # head_dim 256: one workgroup per compute unit
    (8, 2, 72, 16, [900, 300], [800, 299], 4),                     # head_dim 72: the first product's last step half empty
    (6, 2, 40, 32, [700], [650], 3),                               # head_dim 40 in the layout of 64
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached,splits", [
    (32, 8, 128, 16, [1300, 90, 700], [1237, 0, 699], 4),
    (16, 8, 64, 256, [2100, 800], [2000, 512], 5),
    (6, 2, 128, 48, [1000, 30], [900, 7], 3),
])
def test_int8_paged_prefill_split_over_keys(hq, hkv, d, bs, lengths, cached, splits, dtype):
    """The split form over an INT8 cache: against the fp32 oracle over the dequantised cache with the INT8 bounds (2e-2
    beyond the output's half step, mean 2e-3), and against the one-step kernel."""
    from helpers import half_step
    from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8, store_kvcache_int8
    c = make_paged_prefill_case(97, lengths, cached, hq, hkv, d, bs, dtype=dtype, poison=0.0)
    nb = c["k_cache"].shape[0]
    ck, cv = (torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV) for _ in range(2))
    sk, sv = (torch.zeros(nb, bs, hkv, device=DEV) for _ in range(2))
    store_kvcache_int8(c["k_cache"].view(-1, hkv, d).to(DEV), c["v_cache"].view(-1, hkv, d).to(DEV), ck, cv, sk, sv,
                       torch.arange(nb * bs, device=DEV), bs)
    scale = 1 / math.sqrt(d)
    args = (c["q_new"].to(DEV), ck, cv, sk, sv, c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
            hq, hkv, d, bs)
    got = flash_attention_prefill_paged_int8(*args, max_seqlen_k=max(lengths), key_splits=splits).cpu()
    kd = oracle.dequantize_cache_oracle(ck.cpu(), sk.cpu())
    vd = oracle.dequantize_cache_oracle(cv.cpu(), sv.cpu())
    want = oracle.prefill_paged_oracle(c["q_new"].float(), kd, vd, c["block_tables"], c["cu_q"], c["cu_k"], scale,
                                       hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    excess = ((got.float() - want).abs() - half_step(want, dtype)).max().item()
    assert torch.isfinite(got.float()).all() and excess <= 2e-2 and mean <= 2e-3, (mx, excess, mean)
    one_step = flash_attention_prefill_paged_int8(*args).cpu()
    mx, mean = error_stats(got, one_step.float())
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)


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


@pytest.mark.parametrize("seed", range(16))
def test_paged_prefill_split_random_shapes(seed):
    """Seeded random head dims, group sizes, block sizes, range counts, prefixes and bounds on the key count, against
    the one-step form (6600 such cases in a long run differed by at most one bf16 step, 0.0156)."""
    import random
    rng = random.Random(7000 + seed)
    d = rng.choice([128, 128, 64, 80, 32, 96, 256])
    hkv = rng.choice([1, 2, 4, 8])
    hq = hkv * rng.choice([1, 2, 3, 4, 6, 8])
    bs = rng.choice([16, 32, 48, 64, 128, 256])
    nseq = rng.randint(1, 6)
    splits = rng.randint(2, 64 // nseq if nseq > 1 else 40)
    kv, cached = [], []
    for _ in range(nseq):
        c_ = rng.choice([0, rng.randint(0, 200), rng.randint(200, 3000), rng.randint(0, 3000) // 64 * 64])
        kv.append(c_ + rng.choice([1, rng.randint(1, 40), rng.randint(1, 300)]))
        cached.append(c_)
    dtype = rng.choice([torch.bfloat16, torch.float16])
    c = make_paged_prefill_case(8000 + seed, kv, cached, hq, hkv, d, bs, dtype=dtype, poison=0.0)
    scale = 1 / math.sqrt(d)
    one_step = _run(c, hq, hkv, d, bs, scale, 0, None).float()
    got = _run(c, hq, hkv, d, bs, scale, splits, max(kv) + rng.choice([0, 0, 7, 500])).float()
    assert torch.isfinite(got).all()
    mx, mean = error_stats(got, one_step)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (seed, d, hq, hkv, bs, splits, kv, cached, mx, mean)


def test_split_plan_and_rejections():
    from minivllm_amd import _C
    lib = _C.load()
    bf = _C.dtype_code(torch.bfloat16)
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 128, 256, bf, 0) >= 3
    assert lib.mvllm_prefill_paged_split_plan(16, 16384, 2048, 32, 8, 128, 256, bf, 0) == 0      # the chip is full
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 2048, 32, 8, 128, 256, bf, 0) == 0         # too few keys to cut
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 128, 256, bf, 1) >= 3        # INT8 cache
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 80, 256, bf, 1) == 0         # ... not at head_dim 80
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 136, 256, bf, 0) == 0        # head_dim 136: no LDS-tiled kernel
    assert lib.mvllm_prefill_paged_split_plan(1, 128, 32768, 32, 8, 72, 256, bf, 0) > 0          # every multiple of 8 from 32 to 128 has one
    assert lib.mvllm_prefill_paged_split_workspace_bytes(40, 128, 32768, 32, 8, 128, 256, bf, 2) == 0   # 80 ranges
    c = make_paged_prefill_case(5, [300], [200], 8, 8, 128, 16, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        _run(c, 8, 8, 128, 8, 0.1, 4, 300)                        # cache block dimension != block_size
