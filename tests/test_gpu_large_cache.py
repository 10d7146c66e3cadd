"""Caches and packed batches larger than 4 GiB: every kernel addresses them with 64-bit offsets.

Each case runs an operation on a small cache, then on a cache of more than 4 GiB whose last blocks hold the
same data (block ids and slots shifted by the same amount), and asks for bit-identical results: the kernels
do the same arithmetic in the same order wherever the blocks lie.  One case also checks against the CPU oracle.
"""
import math

import pytest
import torch

import oracle
from helpers import error_stats, make_paged_case, make_paged_prefill_case
from minivllm_amd.layers.attention import (flash_attention_prefill, flash_attention_prefill_paged,
                                           paged_attention_decode, paged_attention_decode_int8, store_kvcache,
                                           store_kvcache_int8)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D, BS = 32, 8, 128, 16
FOUR_GIB = 1 << 32


def _big_like(small, num_blocks):
    """Zero cache of `num_blocks` blocks whose last blocks are a copy of `small`; returns (cache, block shift)."""
    big = torch.zeros((num_blocks,) + tuple(small.shape[1:]), dtype=small.dtype, device=DEV)
    shift = num_blocks - small.shape[0]
    big[shift:] = small.to(DEV)
    assert shift * big[0].numel() * big.element_size() > FOUR_GIB
    return big, shift


def _shift_tables(tables, shift):
    return torch.where(tables >= 0, tables + shift, tables).to(torch.int32)


def test_decode_and_paged_prefill_on_blocks_past_4gib():
    nb_big = 140_000                                    # x 32 KiB per block = 4.27 GiB per cache
    q, kc, vc, tables, ctx = make_paged_case(91, 9, 1, 1500, HQ, HKV, D, BS, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(D)
    small = paged_attention_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV), ctx.to(DEV), scale,
                                   HQ, HKV, D, BS)
    want = oracle.decode_naive_oracle(q.float(), kc.float(), vc.float(), tables, ctx, scale, HQ, HKV, D, BS)
    mx, mean = error_stats(small.cpu(), want)
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)
    big_k, shift = _big_like(kc, nb_big)
    big_v, _ = _big_like(vc, nb_big)
    big = paged_attention_decode(q.to(DEV), big_k, big_v, _shift_tables(tables, shift).to(DEV), ctx.to(DEV), scale,
                                 HQ, HKV, D, BS)
    assert torch.equal(small, big)
    del big_k, big_v

    case = make_paged_prefill_case(92, [300, 64, 1000, 17], [128, 0, 512, 16], HQ, HKV, D, BS, dtype=torch.bfloat16)
    args = (case["cu_q"].to(DEV), case["cu_k"].to(DEV), scale, HQ, HKV, D, BS)
    small = flash_attention_prefill_paged(case["q_new"].to(DEV), case["k_cache"].to(DEV), case["v_cache"].to(DEV),
                                          case["block_tables"].to(DEV), *args)
    big_k, shift = _big_like(case["k_cache"], nb_big)
    big_v, _ = _big_like(case["v_cache"], nb_big)
    big = flash_attention_prefill_paged(case["q_new"].to(DEV), big_k, big_v,
                                        _shift_tables(case["block_tables"], shift).to(DEV), *args)
    assert torch.equal(small, big)


def test_store_into_slots_past_4gib():
    nb_big = 140_000
    n = 777
    g = torch.Generator().manual_seed(93)
    key = torch.randn(n, HKV, D, generator=g).to(torch.bfloat16).to(DEV)
    value = torch.randn(n, HKV, D, generator=g).to(torch.bfloat16).to(DEV)
    slots = (nb_big * BS - 1 - torch.randperm(4 * n, generator=g)[:n]).to(torch.int64)   # the last 3108 slots
    slots[5] = -1                                                                   # skipped token
    k_cache = torch.zeros(nb_big, BS, HKV, D, dtype=torch.bfloat16, device=DEV)
    v_cache = torch.zeros_like(k_cache)
    store_kvcache(key, value, k_cache, v_cache, slots.to(DEV), BS)
    live = slots >= 0
    rows_k = k_cache.view(-1, HKV, D)
    rows_v = v_cache.view(-1, HKV, D)
    assert torch.equal(rows_k[slots[live].to(DEV)], key[live.to(DEV)])
    assert torch.equal(rows_v[slots[live].to(DEV)], value[live.to(DEV)])
    assert int(torch.count_nonzero(rows_k[:(nb_big * BS - 4 * n)].view(-1)[::4099])) == 0   # nothing lands low
    tail = rows_k[nb_big * BS - 4 * n:]
    assert int(torch.count_nonzero(tail.abs().sum(dim=(1, 2)))) == int(live.sum())


def test_int8_store_and_decode_past_4gib():
    nb_big = 270_000                                    # x 16 KiB of codes per block = 4.12 GiB per cache
    q, kc, vc, tables, ctx = make_paged_case(94, 6, 1, 900, HQ, HKV, D, BS)
    nb = kc.shape[0]
    scale = 1 / math.sqrt(D)

    def quantise(num_blocks, shift):
        ck = torch.zeros(num_blocks, BS, HKV, D, dtype=torch.int8, device=DEV)
        cv = torch.zeros_like(ck)
        sk = torch.zeros(num_blocks, BS, HKV, device=DEV)
        sv = torch.zeros_like(sk)
        slots = torch.arange(nb * BS, device=DEV) + shift * BS
        store_kvcache_int8(kc.view(-1, HKV, D).to(torch.bfloat16).to(DEV), vc.view(-1, HKV, D).to(torch.bfloat16).to(DEV),
                           ck, cv, sk, sv, slots, BS)
        return ck, cv, sk, sv

    ck, cv, sk, sv = quantise(nb, 0)
    small = paged_attention_decode_int8(q.to(torch.bfloat16).to(DEV), ck, cv, sk, sv, tables.to(DEV), ctx.to(DEV),
                                        scale, HQ, HKV, D, BS)
    shift = nb_big - nb
    assert shift * BS * HKV * D > FOUR_GIB
    bk, bv, bsk, bsv = quantise(nb_big, shift)
    assert torch.equal(bk[shift:], ck) and torch.equal(bv[shift:], cv)
    assert torch.equal(bsk[shift:], sk) and torch.equal(bsv[shift:], sv)
    big = paged_attention_decode_int8(q.to(torch.bfloat16).to(DEV), bk, bv, bsk, bsv,
                                      _shift_tables(tables, shift).to(DEV), ctx.to(DEV), scale, HQ, HKV, D, BS)
    assert torch.equal(small, big)


def test_two_group_prefill_batch_past_4gib():
    """At most 64 sequences (the two-group kernel): 62 long prompts put the last two past the 4 GiB mark of k and v;
    they equal the same two run on their own, bit for bit."""
    lengths = [35400] * 62 + [300, 512]
    total = sum(lengths)
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
    lo = int(cu[62])
    assert lo * HKV * D * 2 > FOUR_GIB
    q = torch.empty(total, HQ, D, dtype=torch.bfloat16, device=DEV)
    k = torch.empty(total, HKV, D, dtype=torch.bfloat16, device=DEV)
    v = torch.empty(total, HKV, D, dtype=torch.bfloat16, device=DEV)
    gen = torch.Generator(device=DEV).manual_seed(96)
    for t in (q, k, v):
        t.normal_(generator=gen)
    scale = 1 / math.sqrt(D)
    out = flash_attention_prefill(q, k, v, cu.to(DEV), scale, HQ, HKV, D)
    torch.cuda.synchronize()
    sub_cu = (cu[62:] - lo).to(torch.int32)
    alone = flash_attention_prefill(q[lo:].clone(), k[lo:].clone(), v[lo:].clone(), sub_cu.to(DEV), scale, HQ, HKV, D)
    assert torch.equal(out[lo:], alone)
    qc, kc, vc = q[lo:lo + 300].cpu(), k[lo:lo + 300].cpu(), v[lo:lo + 300].cpu()
    want = oracle.prefill_standard_oracle(qc.float(), kc.float(), vc.float(), torch.tensor([0, 300], dtype=torch.int32),
                                          scale, HQ, HKV, D)
    mx, mean = error_stats(out[lo:lo + 300].cpu(), want)
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)


def test_packed_prefill_batch_past_4gib():
    """2.2 M packed tokens (K and V 4.5 GiB each, q and the output 18 GiB each): the last sequences equal the same
    sequences run on their own."""
    lengths = [256] * 8600 + [300, 77, 129, 512]
    total = sum(lengths)
    assert total * HKV * D * 2 > FOUR_GIB
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
    q = torch.empty(total, HQ, D, dtype=torch.bfloat16, device=DEV)
    k = torch.empty(total, HKV, D, dtype=torch.bfloat16, device=DEV)
    v = torch.empty(total, HKV, D, dtype=torch.bfloat16, device=DEV)
    gen = torch.Generator(device=DEV).manual_seed(95)
    for t in (q, k, v):
        t.normal_(generator=gen)
    scale = 1 / math.sqrt(D)
    out = flash_attention_prefill(q, k, v, cu.to(DEV), scale, HQ, HKV, D)
    torch.cuda.synchronize()
    lo = int(cu[8599])                                   # the last 5 sequences, all past the 4 GiB mark of k and v
    assert lo * HKV * D * 2 > FOUR_GIB
    sub_cu = (cu[8599:] - lo).to(torch.int32)
    alone = flash_attention_prefill(q[lo:].clone(), k[lo:].clone(), v[lo:].clone(), sub_cu.to(DEV), scale, HQ, HKV, D)
    # more than 64 sequences run on prefill_mfma_kernel, the five alone on the two-group kernel (row sums taken before
    # the weights are rounded): equal to the last bits of the 16-bit outputs, which no wrong address would be
    err = (out[lo:].float() - alone.float()).abs()
    assert (err <= alone.float().abs() * 2.0 ** -6 + 1e-3).all() and err.mean() <= 2e-4
    # and the very first sequence against the oracle
    qc, kc, vc = q[:256].cpu(), k[:256].cpu(), v[:256].cpu()
    want = oracle.prefill_standard_oracle(qc.float(), kc.float(), vc.float(), torch.tensor([0, 256], dtype=torch.int32),
                                          scale, HQ, HKV, D)
    mx, mean = error_stats(out[:256].cpu(), want)
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)


def test_fused_qk_store_into_slots_past_4gib():
    """qk_norm_rope_store writes the same rows whether the slots lie at the start or past 4 GiB of the cache."""
    from minivllm_amd.layers.fused import qk_norm_rope_store
    nb_big, nb_small, t = 140_000, 8, 100
    g = torch.Generator().manual_seed(96)
    qkv = torch.randn(t, (HQ + 2 * HKV) * D, generator=g).to(torch.bfloat16).to(DEV)
    q, k, v = qkv.split([HQ * D, HKV * D, HKV * D], dim=-1)
    q, k, v = q.unflatten(-1, (HQ, D)), k.unflatten(-1, (HKV, D)), v.unflatten(-1, (HKV, D))
    pos = torch.randint(0, 512, (t,), generator=g).to(DEV)
    gamma = (torch.rand(D, generator=g) + 0.5).float().to(DEV)
    table = oracle.rope_cos_sin_cache_oracle(1e6, D, 512).to(DEV)
    slots = torch.randperm(nb_small * BS, generator=g)[:t].to(torch.int64)
    results = []
    for num_blocks in (nb_small, nb_big):
        shift = (num_blocks - nb_small) * BS
        kc = torch.zeros(num_blocks, BS, HKV, D, dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros_like(kc)
        out = qk_norm_rope_store(q, k, v, pos, table, gamma, 1e-6, (slots + shift).to(DEV), kc, vc)
        results.append((out, kc[num_blocks - nb_small:].clone(), vc[num_blocks - nb_small:].clone()))
        if shift:
            assert shift * HKV * D * 2 > FOUR_GIB
            assert int(torch.count_nonzero(kc[:num_blocks - nb_small].view(-1)[::4099])) == 0
        del kc, vc
    (out_a, k_a, v_a), (out_b, k_b, v_b) = results
    assert all(torch.equal(a, b) for a, b in zip(out_a, out_b))
    assert torch.equal(k_a, k_b) and torch.equal(v_a, v_b)
    assert torch.equal(k_a.view(-1, HKV, D)[slots.to(DEV)], out_a[1])       # the rotated keys are what was stored
