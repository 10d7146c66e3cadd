"""Seeded random shapes over every head_dim the MFMA kernels take, through the attention entry points on the GPU against
the CPU oracle (test_gpu_random_shapes.py does the same at head_dim 128 with empty contexts): head dims, head counts up
to 24 query heads per kv head, block sizes, batch sizes up to 70 sequences and lengths drawn together, so that
combinations nobody wrote a case for still get checked (a single short sequence behind a long prefix on the kernel
with 128-row items was found this way).  Small sizes, so that the oracle stays fast; tolerances as in the per-operator
tests (bf16 / fp16: max-abs <= 2e-2, mean-abs <= 2e-3)."""
import math

import pytest
import torch

import oracle
from helpers import error_stats, make_paged_case, make_paged_prefill_case, make_varlen_case
from minivllm_amd.layers.attention import (flash_attention_prefill, flash_attention_prefill_paged,
                                           paged_attention_decode)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16 = 2e-2, 2e-3
HEAD_DIMS = [32, 40, 48, 56, 64, 72, 80, 88, 96, 104, 112, 120, 128, 128, 128, 128, 256]   # every MFMA head dim


def _pick(g, xs):
    return xs[int(torch.randint(0, len(xs), (1,), generator=g))]


def _shape(g):
    d = _pick(g, HEAD_DIMS)
    hkv = _pick(g, [1, 2, 3, 4, 8])
    group = _pick(g, [1, 2, 3, 4, 5, 6, 8, 10, 16, 17, 24])
    while hkv * group * d > 8192:
        hkv = max(1, hkv // 2)
        group = max(1, group // 2)
    return hkv * group, hkv, d, _pick(g, [torch.bfloat16, torch.float16])


def _lengths(g, num_seqs, top):
    out = [int(torch.randint(0, top + 1, (1,), generator=g)) if int(torch.randint(0, 8, (1,), generator=g)) else 0
           for _ in range(num_seqs)]
    if sum(out) == 0:
        out[0] = 5
    return out


@pytest.mark.parametrize("seed", range(8))
def test_random_packed_prefill(seed):
    g = torch.Generator().manual_seed(4100 + seed)
    for case in range(12):
        hq, hkv, d, dtype = _shape(g)
        num_seqs = _pick(g, [1, 2, 3, 8, 20, 70])
        lengths = _lengths(g, num_seqs, _pick(g, [70, 200, 500]) if num_seqs <= 8 else _pick(g, [40, 130]))
        q, k, v, cu = make_varlen_case(4200 + 16 * seed + case, lengths, hq, hkv, d, dtype=dtype)
        scale = 1 / math.sqrt(d)
        got = flash_attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), scale, hq, hkv, d).cpu()
        want = oracle.prefill_standard_oracle(q.float(), k.float(), v.float(), cu, scale, hq, hkv, d)
        mx, mean = error_stats(got, want)
        what = (hq, hkv, d, dtype, lengths[:8], num_seqs)
        assert torch.isfinite(got.float()).all() and mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (what, mx, mean)


@pytest.mark.parametrize("seed", range(8))
def test_random_paged_prefill(seed):
    g = torch.Generator().manual_seed(4300 + seed)
    for case in range(12):
        hq, hkv, d, dtype = _shape(g)
        bs = _pick(g, [16, 32, 48, 256])
        num_seqs = _pick(g, [1, 1, 2, 3, 8, 20])
        new = _lengths(g, num_seqs, _pick(g, [5, 70, 200]) if num_seqs <= 8 else _pick(g, [5, 40]))
        cached = [_pick(g, [0, int(torch.randint(0, 300, (1,), generator=g)), 64 * int(torch.randint(0, 5, (1,), generator=g)),
                            int(torch.randint(0, 1900, (1,), generator=g))]) for _ in range(num_seqs)]
        kv = [a + b for a, b in zip(new, cached)]
        c = make_paged_prefill_case(4400 + 16 * seed + case, kv, cached, hq, hkv, d, bs, dtype=dtype)
        scale = 1 / math.sqrt(d)
        got = flash_attention_prefill_paged(c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV),
                                            c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
                                            hq, hkv, d, bs).cpu()
        want = oracle.prefill_paged_oracle(c["q_new"].float(), c["k_cache"].float(), c["v_cache"].float(),
                                           c["block_tables"], c["cu_q"], c["cu_k"], scale, hq, hkv, d, bs)
        mx, mean = error_stats(got, want)
        what = (hq, hkv, d, bs, dtype, new[:8], cached[:8], num_seqs)
        assert torch.isfinite(got.float()).all() and mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (what, mx, mean)


@pytest.mark.parametrize("seed", range(8))
def test_random_decode(seed):
    g = torch.Generator().manual_seed(4500 + seed)
    for case in range(12):
        hq, hkv, d, dtype = _shape(g)
        bs = _pick(g, [16, 32, 64, 256])
        batch = _pick(g, [1, 2, 7, 16, 64])
        top = _pick(g, [5, 100, 700, 2500]) if batch <= 16 else _pick(g, [5, 100, 400])
        ctx_list = [int(torch.randint(1, top + 1, (1,), generator=g)) for _ in range(batch)]
        q, kc, vc, tables, ctx = make_paged_case(4600 + 16 * seed + case, 0, 0, 0, hq, hkv, d, bs, dtype=dtype,
                                                 ctx_list=ctx_list)
        scale = 1 / math.sqrt(d)
        got = paged_attention_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV), ctx.to(DEV), scale, hq, hkv, d,
                                     bs).cpu()
        want = oracle.decode_vectorised_oracle(q.float(), kc.float(), vc.float(), tables, ctx, scale, hq, hkv, d, bs)
        mx, mean = error_stats(got, want)
        what = (hq, hkv, d, bs, dtype, batch, ctx_list[:8])
        assert torch.isfinite(got.float()).all() and mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (what, mx, mean)
