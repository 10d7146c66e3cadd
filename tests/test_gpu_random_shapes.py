"""Seeded random shapes through the three attention entry points against the CPU oracle: head counts, group
sizes, block sizes, context lengths (zero included) and prompt lengths drawn per case, so that paths the
hand-picked cases do not name (odd groups, tiny partitions, empty sequences in the middle of a batch) are
walked too.  Tolerances as in the other GPU tests."""
import math
import random

import pytest
import torch

import oracle
from helpers import error_stats, make_paged_case, make_paged_prefill_case, make_varlen_case
from minivllm_amd.layers.attention import (flash_attention_prefill, flash_attention_prefill_paged,
                                            paged_attention_decode)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16 = 2e-2, 2e-3
D = 128


def _heads(rng):
    hkv = rng.choice([1, 2, 3, 4, 8])
    group = rng.choice([1, 2, 3, 4, 5, 8, 12, 16])
    return hkv * group, hkv


@pytest.mark.parametrize("seed", range(12))
def test_decode_random_shapes(seed):
    rng = random.Random(1000 + seed)
    hq, hkv = _heads(rng)
    bs = rng.choice([16, 32, 48, 64, 256])
    batch = rng.randint(1, 9)
    hi = rng.choice([40, 300, 1200, 2600])
    ctx = [rng.randint(0, hi) for _ in range(batch)]
    ctx[rng.randrange(batch)] = max(ctx[0], 1)           # at least one non-empty sequence
    dtype = rng.choice([torch.bfloat16, torch.float16])
    q, kc, vc, tables, ctx_t = make_paged_case(2000 + seed, batch, 0, 0, hq, hkv, D, bs, dtype=dtype, ctx_list=ctx)
    scale = 1 / math.sqrt(D)
    got = paged_attention_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV),
                                 ctx_t.to(rng.choice([torch.int32, torch.int64])).to(DEV), scale, hq, hkv, D, bs).cpu()
    assert torch.isfinite(got).all()
    for b in range(batch):
        if ctx[b] == 0:
            assert got[b].abs().max() == 0                # an empty context gives a row of zeros
            continue
        want = oracle.decode_naive_oracle(q[b:b + 1].float(), kc.float(), vc.float(), tables[b:b + 1],
                                          ctx_t[b:b + 1], scale, hq, hkv, D, bs)
        mx, mean = error_stats(got[b:b + 1], want)
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (seed, b, hq, hkv, bs, ctx[b], mx, mean)


@pytest.mark.parametrize("seed", range(10))
def test_prefill_random_shapes(seed):
    rng = random.Random(3000 + seed)
    hkv = rng.choice([1, 2, 4, 8])
    hq = hkv * rng.choice([1, 2, 4, 8])                   # the groups the MFMA kernel takes, and via 8 two chunks
    n = rng.randint(1, 7)
    lengths = [rng.choice([0, 1, rng.randint(2, 70), rng.randint(71, 400)]) for _ in range(n)]
    if sum(lengths) == 0:
        lengths[0] = 33
    dtype = rng.choice([torch.bfloat16, torch.float16])
    q, k, v, cu = make_varlen_case(4000 + seed, lengths, hq, hkv, D, dtype=dtype)
    scale = 1 / math.sqrt(D)
    got = flash_attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), scale, hq, hkv, D).cpu()
    want = oracle.prefill_standard_oracle(q.float(), k.float(), v.float(), cu, scale, hq, hkv, D)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (seed, hq, hkv, lengths, mx, mean)


@pytest.mark.parametrize("seed", range(8))
def test_paged_prefill_random_shapes(seed):
    rng = random.Random(5000 + seed)
    hkv = rng.choice([1, 2, 4, 8])
    hq = hkv * rng.choice([1, 2, 4])
    bs = rng.choice([16, 32, 64, 256])
    n = rng.randint(1, 5)
    kv = [rng.randint(1, 420) for _ in range(n)]
    cached = [rng.choice([0, (L - 1) // bs * bs, rng.randint(0, L - 1)]) for L in kv]   # at least one new token each
    c = make_paged_prefill_case(6000 + seed, kv, cached, hq, hkv, D, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(D)
    got = flash_attention_prefill_paged(c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV),
                                        c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
                                        hq, hkv, D, bs).cpu()
    want = oracle.prefill_paged_oracle(c["q_new"].float(), torch.nan_to_num(c["k_cache"].float()),
                                       torch.nan_to_num(c["v_cache"].float()), c["block_tables"], c["cu_q"],
                                       c["cu_k"], scale, hq, hkv, D, bs)
    assert torch.isfinite(got).all()
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (seed, hq, hkv, bs, kv, cached, mx, mean)
