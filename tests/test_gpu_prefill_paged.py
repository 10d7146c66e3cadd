"""flash_attention_prefill_paged (prefill after a cached prefix, keys from the paged cache) on the GPU vs the CPU
oracle; tolerances as for the plain prefill: bf16/fp16 max-abs <= 2e-2 and mean-abs <= 2e-3, fp32 max-abs <= 2e-4,
against the oracle evaluated in fp32 on the same inputs.  Cache rows past a sequence's end hold NaN in these
cases: any leak shows up as NaN in the output."""
import math

import pytest
import torch

import oracle
from helpers import error_stats, half_step, make_paged_prefill_case
from minivllm_amd.layers.attention import (Attention, flash_attention_prefill, flash_attention_prefill_paged,
                                           paged_attention_decode)
from minivllm_amd.utils import reset_context, set_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16, MAX_ABS_32 = 2e-2, 2e-3, 2e-4


def _run(c, scale, hq, hkv, d, bs):
    out = flash_attention_prefill_paged(c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV),
                                        c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
                                        hq, hkv, d, bs)
    torch.cuda.synchronize()
    return out.cpu()


def _oracle32(c, scale, hq, hkv, d, bs):
    return oracle.prefill_paged_oracle(c["q_new"].float(), c["k_cache"].float(), c["v_cache"].float(),
                                       c["block_tables"], c["cu_q"], c["cu_k"], scale, hq, hkv, d, bs)


def _check(got, want, dtype):
    assert not torch.isnan(got.float()).any()
    mx, mean = error_stats(got, want)
    if dtype == torch.float32:
        assert mx <= MAX_ABS_32, mx
    else:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached", [
    (32, 8, 128, 16, [300, 64, 129, 500], [256, 0, 16, 48]),       # prefixes at multiples of 16, 64-aligned or not
    (32, 8, 128, 256, [700, 300, 257], [512, 256, 0]),             # the engine's block size
    (16, 8, 128, 16, [200, 90], [160, 80]),                        # GQA 2
    (8, 8, 128, 32, [150], [96]),                                  # no grouping
    (32, 8, 128, 16, [131, 77, 260], [50, 1, 259]),                # prefixes at arbitrary token counts, 1 new token
    (6, 2, 80, 8, [40, 23], [16, 8]),                              # generic kernel (head_dim 80)
    (8, 2, 96, 16, [300, 64, 129], [256, 0, 17]),                  # head_dim 96 in the 128 layout: the tiled kernel
    (6, 3, 112, 32, [131, 260], [50, 259]),                        # head_dim 112, two query heads per kv head
    (4, 4, 32, 16, [200, 70], [160, 32]),                          # head_dim 32 in the 64 layout
    (8, 2, 80, 16, [140, 23], [16, 8]),                            # head_dim 80, blocks of 16: the tiled kernel
    (8, 2, 256, 16, [300, 64, 129], [256, 0, 17]),                 # head_dim 256: 512-byte tile rows
    (8, 2, 72, 16, [300, 64, 129], [256, 0, 17]),                  # head_dim 72: the first product's last step half empty (fp32: generic)
    (6, 3, 120, 32, [131, 260], [50, 259]),                        # head_dim 120
    (4, 4, 40, 16, [200, 70], [160, 32]),                          # head_dim 40 in the 64 layout
    (4, 4, 64, 16, [70], [32]),                                    # head_dim 64: 16-row tiles (fp32: generic kernel)
    (16, 8, 64, 16, [300, 64, 129, 500], [256, 0, 17, 48]),        # head_dim 64, the reference demo's heads
    (12, 1, 64, 256, [700, 30, 257], [512, 29, 0]),                # head_dim 64, one kv head, the engine's block size
    (6, 2, 64, 48, [131, 77, 260], [50, 1, 259]),                  # head_dim 64, heads not a multiple of four
    (4, 4, 64, 8, [70], [32]),                                     # head_dim 64 with a block size of 8: generic kernel
    (6, 2, 128, 16, [131, 77, 260], [50, 1, 259]),                 # head_dim 128, three query heads per kv head (one head per workgroup)
])
def test_paged_prefill_vs_oracle(dtype, hq, hkv, d, bs, lengths, cached):
    c = make_paged_prefill_case(61, lengths, cached, hq, hkv, d, bs, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(c, scale, hq, hkv, d, bs)
    want = _oracle32(c, scale, hq, hkv, d, bs)
    assert got.dtype == dtype and got.shape == want.shape
    _check(got, want, dtype)


def test_paged_prefill_without_prefix_matches_plain_prefill_bitwise():
    """No cached prefix: same tiles, same arithmetic as the packed kernel, only the copies' source differs.  (Three query
    heads per kv head: both calls run on prefill_mfma_kernel.)"""
    hq, hkv, d, bs = 24, 8, 128, 16
    lengths = [257, 64, 31, 400]
    c = make_paged_prefill_case(62, lengths, [0] * 4, hq, hkv, d, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    got = _run(c, scale, hq, hkv, d, bs)
    plain = flash_attention_prefill(c["q"].to(DEV), c["k"].to(DEV), c["v"].to(DEV), c["cu_k"].to(DEV), scale,
                                    hq, hkv, d).cpu()
    assert torch.equal(got, plain)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (16, 8)])
@pytest.mark.parametrize("bs", [16, 48, 256])
def test_two_group_paged_prefill_without_prefix_matches_packed_bitwise(bs, hq, hkv):
    """Four (or two) query heads per kv head: both calls run on the two-group kernel, same tiles, same arithmetic, only
    the copies' source differs (the paged cache through the block table)."""
    d = 128
    lengths = [257, 64, 31, 400, 1, 1000]
    c = make_paged_prefill_case(62, lengths, [0] * 6, hq, hkv, d, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    got = _run(c, scale, hq, hkv, d, bs)
    plain = flash_attention_prefill(c["q"].to(DEV), c["k"].to(DEV), c["v"].to(DEV), c["cu_k"].to(DEV), scale,
                                    hq, hkv, d).cpu()
    assert torch.equal(got, plain)


def test_paged_prefill_single_new_token_matches_decode():
    hq, hkv, d, bs = 32, 8, 128, 16
    lengths = [300, 17, 1, 64]
    c = make_paged_prefill_case(63, lengths, [n - 1 for n in lengths], hq, hkv, d, bs, dtype=torch.bfloat16,
                                poison=0.0)
    scale = 1 / math.sqrt(d)
    got = _run(c, scale, hq, hkv, d, bs)
    dec = paged_attention_decode(c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV),
                                 c["block_tables"].to(DEV), torch.tensor(lengths, device=DEV), scale, hq, hkv, d,
                                 bs).cpu()
    mx, mean = error_stats(got, dec.float())
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16


def test_paged_prefill_unmapped_blocks_and_empty_sequences():
    """A table entry outside the pool is not followed: its keys and values read as zeros, exactly as if the
    entry pointed at a block of zeros.  A sequence without new tokens produces no rows."""
    hq, hkv, d, bs = 8, 2, 128, 16
    lengths, cached = [100, 40, 70], [32, 40, 0]                   # the second sequence has no new tokens
    for dtype in (torch.bfloat16, torch.float32):
        c = make_paged_prefill_case(64, lengths, cached, hq, hkv, d, bs, dtype=dtype)
        zero_block = c["k_cache"].shape[0]
        kc = torch.cat([c["k_cache"], torch.zeros(1, bs, hkv, d, dtype=dtype)])
        vc = torch.cat([c["v_cache"], torch.zeros(1, bs, hkv, d, dtype=dtype)])
        want_tables = c["block_tables"].clone()
        want_tables[0, 1] = zero_block                             # oracle: the hole is a block of zeros
        want = _oracle32(dict(c, k_cache=kc, v_cache=vc, block_tables=want_tables), 0.09, hq, hkv, d, bs)
        for bad in (-1, 10 ** 6):
            c["block_tables"][0, 1] = bad
            got = _run(c, 0.09, hq, hkv, d, bs)
            _check(got, want, dtype)
        assert int(c["cu_q"][2] - c["cu_q"][1]) == 0 and got.shape[0] == 68 + 70


@pytest.mark.parametrize("bs", [16, 8])
def test_attention_module_uses_the_paged_prefill_when_block_tables_are_set(bs):
    """Store the new tokens, then prefill over (cached prefix + new tokens) through ``Attention.forward``, as the
    engine does on a prefix-cache hit.  With 8 tokens per block the module's max_seqlen_k sends the call through the
    two-step form (a temporary cache of 16-token blocks)."""
    hq, hkv, d = 16, 8, 128
    lengths, cached = [120, 50], [64, 16]
    c = make_paged_prefill_case(65, lengths, cached, hq, hkv, d, bs, dtype=torch.bfloat16, poison=0.0)
    att = Attention(hq, d, 1.0, hkv, bs)
    kc, vc = c["k_cache"].clone(), c["v_cache"].clone()
    slots = torch.cat([torch.tensor([int(c["block_tables"][s, j // bs]) * bs + j % bs
                                     for j in range(cached[s], lengths[s])]) for s in range(2)])
    kc.view(-1, hkv, d)[slots] = 0                                  # the new tokens are not in the cache yet
    vc.view(-1, hkv, d)[slots] = 0
    att.k_cache, att.v_cache = kc.to(DEV), vc.to(DEV)
    k_new, v_new = c["k"][c["new_rows"]], c["v"][c["new_rows"]]
    set_context(True, c["cu_q"].to(DEV), c["cu_k"].to(DEV), 64, 128, slots.to(DEV), None, c["block_tables"].to(DEV))
    try:
        out = att(c["q_new"].to(DEV), k_new.to(DEV), v_new.to(DEV)).cpu()
    finally:
        reset_context()
    want = _oracle32(c, 1 / math.sqrt(d), hq, hkv, d, bs).reshape(out.shape[0], -1)
    mx, mean = error_stats(out, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16


@pytest.mark.parametrize("hq,hkv,d,bs", [(16, 8, 64, 16), (8, 2, 72, 16), (6, 6, 40, 32), (8, 4, 256, 16), (6, 2, 120, 64)])
def test_paged_prefill_other_head_dims_without_prefix_match_plain_prefill_bitwise(hq, hkv, d, bs):
    """The one-group kernel's paged and packed forms at head_dim 64, at head dims whose last 16-dim step is half empty
    (72, 40, 120) and at 256: same tiles, same arithmetic, only the copies' source differs."""
    c = make_paged_prefill_case(66, [90, 1, 257, 33], [0, 0, 0, 0], hq, hkv, d, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    plain = flash_attention_prefill(c["q"].to(DEV), c["k"].to(DEV), c["v"].to(DEV), c["cu_k"].to(DEV), scale, hq, hkv, d).cpu()
    assert torch.equal(_run(c, scale, hq, hkv, d, bs), plain)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached", [
    (32, 8, 128, 16, [300, 64, 129, 500], [256, 0, 17, 48]),
    (16, 8, 64, 16, [200, 90, 33], [160, 80, 0]),                  # the reference demo's heads
    (12, 1, 128, 256, [700, 30, 257], [512, 29, 0]),               # one kv head, the engine's block size
    (6, 2, 64, 48, [131, 77, 260], [50, 1, 259]),                  # three query heads per kv head
])
def test_paged_prefill_over_an_int8_cache(dtype, hq, hkv, d, bs, lengths, cached):
    """Every key comes from the INT8 cache: the oracle is the paged prefill over the dequantised cache (code * scale
    in fp32).  Mean-abs 2e-3; max-abs 2e-2 beyond half a step of the output type at the value (see
    test_int8_paged_prefill_short_sequences for why that half step is there)."""
    from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8, store_kvcache_int8
    c = make_paged_prefill_case(67, lengths, cached, hq, hkv, d, bs, dtype=dtype, poison=0.0)
    nb = c["k_cache"].shape[0]
    ck, cv = (torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV) for _ in range(2))
    sk, sv = (torch.zeros(nb, bs, hkv, device=DEV) for _ in range(2))
    store_kvcache_int8(c["k_cache"].view(-1, hkv, d).to(DEV), c["v_cache"].view(-1, hkv, d).to(DEV), ck, cv, sk, sv,
                       torch.arange(nb * bs, device=DEV), bs)
    scale = 1 / math.sqrt(d)
    got = flash_attention_prefill_paged_int8(c["q_new"].to(DEV), ck, cv, sk, sv, c["block_tables"].to(DEV),
                                             c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale, hq, hkv, d, bs).cpu()
    kd = oracle.dequantize_cache_oracle(ck.cpu(), sk.cpu())
    vd = oracle.dequantize_cache_oracle(cv.cpu(), sv.cpu())
    want = oracle.prefill_paged_oracle(c["q_new"].float(), kd, vd, c["block_tables"], c["cu_q"], c["cu_k"], scale,
                                       hq, hkv, d, bs)
    assert got.dtype == dtype and got.shape == want.shape and torch.isfinite(got.float()).all()
    mx, mean = error_stats(got, want)
    excess = ((got.float() - want).abs() - half_step(want, dtype)).max().item()
    assert excess <= 2e-2 and mean <= 2e-3, (mx, excess, mean)
    # one new token per sequence: the same rows as INT8 decode over the same cache
    from minivllm_amd.layers.attention import paged_attention_decode_int8
    last = torch.tensor([int(c["cu_q"][i + 1]) - 1 for i in range(len(lengths))])
    dec = paged_attention_decode_int8(c["q_new"][last].to(DEV), ck, cv, sk, sv, c["block_tables"].to(DEV),
                                      torch.tensor(lengths, device=DEV), scale, hq, hkv, d, bs).cpu()
    mx, mean = error_stats(got[last], dec.float())
    assert mx <= 3e-2 and mean <= 3e-3, (mx, mean)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (64, 8), (8, 2), (12, 3), (16, 8), (12, 2), (2, 1)])
@pytest.mark.parametrize("bs", [16, 48, 256])
@pytest.mark.parametrize("num_seqs", [1, 9, 64])
def test_two_group_paged_prefill_takes_every_item_once(hq, hkv, bs, num_seqs):
    """The two-group kernel over cached prefixes (head_dim 128, an even number of query heads per kv head, at most 64
    sequences; items of four heads and 64 rows, or with 2 / 6 heads per kv head of two heads and 128 rows): prefixes of
    0, whole tiles and anything in between (the diagonal then crosses one tile more at an item's end), a single new
    token behind a long prefix, sequences with nothing new, blocks of 16, 48 and 256 tokens in shuffled physical order
    with poisoned rows past every sequence's end.  The output starts as NaN, so an item that no workgroup took would
    show."""
    d = 128
    g = torch.Generator().manual_seed(1300 + num_seqs + bs + hq)
    pool = [1, 2, 31, 63, 64, 65, 100, 128, 129, 191, 192, 257, 300, 448]
    kv_lengths = [pool[i] for i in torch.randint(0, len(pool), (num_seqs,), generator=g).tolist()]
    kv_lengths[num_seqs // 2] = 1500 if hq <= 32 else 600
    cached = []
    for n in kv_lengths:
        mode = int(torch.randint(0, 5, (1,), generator=g))
        c = [0, n - 1, (n // 2) // 64 * 64, n // 2, n][mode]      # nothing, all but one, whole tiles, half, everything
        cached.append(max(0, min(c, n)))
    cached[num_seqs // 2] = 333                                    # the long one: a prefix that ends inside a tile
    if sum(n - c for n, c in zip(kv_lengths, cached)) == 0:
        cached[0] = 0
    c = make_paged_prefill_case(70, kv_lengths, cached, hq, hkv, d, bs, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    from minivllm_amd import _C
    q_new = c["q_new"].to(DEV)
    out = torch.full_like(q_new, float("nan"))
    kc, vc, bt, cuq, cuk = (c[k].to(DEV) for k in ("k_cache", "v_cache", "block_tables", "cu_q", "cu_k"))
    st = _C.load().mvllm_prefill_paged(out.data_ptr(), q_new.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(),
                                       bt.shape[1], cuq.data_ptr(), cuk.data_ptr(), num_seqs, q_new.shape[0], hq, hkv, d, bs,
                                       kc.shape[0], scale, _C.dtype_code(q_new.dtype), _C.current_stream_ptr(out.device))
    torch.cuda.synchronize()
    assert st == 0
    _check(out.cpu(), _oracle32(c, scale, hq, hkv, d, bs), torch.bfloat16)


def _int8_case(seed, lengths, cached, hq, hkv, d, bs, dtype):
    from minivllm_amd.layers.attention import store_kvcache_int8
    c = make_paged_prefill_case(seed, lengths, cached, hq, hkv, d, bs, dtype=dtype, poison=0.0)
    nb = c["k_cache"].shape[0]
    ck, cv = (torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV) for _ in range(2))
    sk, sv = (torch.zeros(nb, bs, hkv, device=DEV) for _ in range(2))
    store_kvcache_int8(c["k_cache"].view(-1, hkv, d).to(DEV), c["v_cache"].view(-1, hkv, d).to(DEV), ck, cv, sk, sv,
                       torch.arange(nb * bs, device=DEV), bs)
    return c, ck, cv, sk, sv


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached,slack", [
    (32, 8, 128, 16, [300, 64, 129, 500], [256, 0, 17, 48], 0),
    (16, 8, 128, 256, [700, 30, 257], [512, 29, 0], 5),                 # two query heads per kv head, the engine's block size
    (12, 2, 128, 48, [131, 77, 260, 1, 90], [50, 1, 259, 0, 90], 100),  # six heads per kv head; a sequence with nothing new
    (8, 2, 128, 32, [1500], [1499], 0),                                 # one new token behind a long prefix
    (6, 2, 128, 16, [131, 77, 260], [50, 1, 259], 3),                   # three heads per kv head: the one-group kernel
    (16, 8, 64, 16, [200, 90, 33], [160, 80, 0], 0),                    # head_dim 64: the one-group kernel
])
def test_int8_paged_prefill_in_two_steps(dtype, hq, hkv, d, bs, lengths, cached, slack):
    """With max_seqlen_k the INT8 prefill stages the batch's keys and values as 16-bit values in a temporary cache of
    16-token blocks and runs the two-group kernel (shapes it does not take: the one-group kernel) over it.  The staged
    values are the oracle's code * scale rounded
    to the query type, so the result equals, bit for bit, the 16-bit paged prefill over a cache holding exactly those
    values (whatever its block size), and it meets the INT8 bounds against the fp32 oracle.  max_seqlen_k may be any
    upper bound of the key counts."""
    from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8
    from minivllm_amd import _C
    c, ck, cv, sk, sv = _int8_case(72, lengths, cached, hq, hkv, d, bs, dtype)
    scale = 1 / math.sqrt(d)
    top = max(lengths) + slack
    assert _C.load().mvllm_prefill_paged_staged_workspace_bytes(len(lengths), top, hq, hkv, d, _C.dtype_code(dtype), 1) > 0
    args = (c["q_new"].to(DEV), ck, cv, sk, sv, c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale,
            hq, hkv, d, bs)
    got = flash_attention_prefill_paged_int8(*args, max_seqlen_k=top).cpu()
    kd = oracle.dequantize_cache_oracle(ck.cpu(), sk.cpu())
    vd = oracle.dequantize_cache_oracle(cv.cpu(), sv.cpu())
    same = flash_attention_prefill_paged(c["q_new"].to(DEV), kd.to(dtype).to(DEV), vd.to(dtype).to(DEV),
                                         c["block_tables"].to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale, hq, hkv,
                                         d, bs).cpu()
    assert torch.equal(got, same)
    want = oracle.prefill_paged_oracle(c["q_new"].float(), kd, vd, c["block_tables"], c["cu_q"], c["cu_k"], scale,
                                       hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    excess = ((got.float() - want).abs() - half_step(want, dtype)).max().item()
    assert torch.isfinite(got.float()).all() and excess <= 2e-2 and mean <= 2e-3, (mx, excess, mean)
    one_step = flash_attention_prefill_paged_int8(*args).cpu()                # the one-step kernel: same values, other order
    mx, mean = error_stats(got, one_step.float())
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)


def test_int8_paged_prefill_in_two_steps_unmapped_block_and_unsupported_shapes():
    """A table entry outside the pool stages zeros, as the one-step kernel reads them; shapes the MFMA kernels do not
    take report no workspace and the operator runs in one step."""
    from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8
    from minivllm_amd import _C
    hq, hkv, d, bs, dtype = 8, 2, 128, 16, torch.bfloat16
    lengths, cached = [100, 70], [32, 0]
    c, ck, cv, sk, sv = _int8_case(73, lengths, cached, hq, hkv, d, bs, dtype)
    tables = c["block_tables"].clone()
    tables[0, 1] = 10 ** 6
    args = (c["q_new"].to(DEV), ck, cv, sk, sv, tables.to(DEV), c["cu_q"].to(DEV), c["cu_k"].to(DEV), 0.09, hq, hkv, d, bs)
    got = flash_attention_prefill_paged_int8(*args, max_seqlen_k=100).cpu()
    one_step = flash_attention_prefill_paged_int8(*args).cpu()
    mx, mean = error_stats(got, one_step.float())
    assert torch.isfinite(got.float()).all() and mx <= 2e-2 and mean <= 2e-3, (mx, mean)
    ws = _C.load().mvllm_prefill_paged_staged_workspace_bytes
    code = _C.dtype_code(dtype)
    assert ws(2, 100, hq, hkv, d, code, 1) == 2 * (2 * 7 * 16 * hkv * d * 2) + 256 == ws(2, 100, hq, hkv, d, code, 0)
    assert ws(2, 100, 6, 2, d, code, 1) > 0 and ws(2, 100, hq, hkv, 64, code, 1) > 0 and ws(65, 100, hq, hkv, d, code, 1) > 0
    assert ws(2, 100, hq, hkv, 96, code, 1) == 0 and ws(2, 100, hq, hkv, 96, code, 0) > 0      # head_dim 96: 16-bit caches only
    assert ws(2, 100, hq, hkv, 136, code, 0) == 0 and ws(2, 100, hq, hkv, 100, code, 0) == 0    # no LDS-tiled kernel for these
    assert ws(2, 100, hq, hkv, 72, code, 0) > 0                                                  # 16-bit cache, any multiple of 8 from 32 to 128
    assert ws(2, 100, hq, hkv, d, _C.dtype_code(torch.float32), 1) == 0 and ws(2, 0, hq, hkv, d, code, 1) == 0
    # block size 8: the one-step INT8 kernels do not take it, the two-step form does
    c8, ck8, cv8, sk8, sv8 = _int8_case(74, lengths, cached, hq, hkv, d, 8, dtype)
    args8 = (c8["q_new"].to(DEV), ck8, cv8, sk8, sv8, c8["block_tables"].to(DEV), c8["cu_q"].to(DEV), c8["cu_k"].to(DEV),
             0.09, hq, hkv, d, 8)
    with pytest.raises(ValueError):
        flash_attention_prefill_paged_int8(*args8)
    got8 = flash_attention_prefill_paged_int8(*args8, max_seqlen_k=100).cpu()
    kd = oracle.dequantize_cache_oracle(ck8.cpu(), sk8.cpu())
    vd = oracle.dequantize_cache_oracle(cv8.cpu(), sv8.cpu())
    want8 = oracle.prefill_paged_oracle(c8["q_new"].float(), kd, vd, c8["block_tables"], c8["cu_q"], c8["cu_k"], 0.09,
                                        hq, hkv, d, 8)
    mx, mean = error_stats(got8, want8)
    excess = ((got8.float() - want8).abs() - half_step(want8, dtype)).max().item()
    assert excess <= 2e-2 and mean <= 2e-3, (mx, excess, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,bs,lengths,cached", [
    (32, 8, 128, 8, [300, 64, 129, 500], [256, 0, 17, 48]),        # block size 8: the two-group kernel over the staged cache
    (16, 8, 128, 1, [200, 90, 33], [160, 80, 0]),                  # a block per token
    (6, 2, 128, 24, [131, 77, 260], [50, 1, 259]),                 # 24 tokens per block, three query heads per kv head
    (16, 8, 64, 8, [200, 90, 33, 5], [160, 80, 0, 5]),             # head_dim 64; a sequence with nothing new
    (6, 2, 96, 3, [131, 77], [50, 1]),                             # head_dim 96, 3 tokens per block
])
def test_paged_prefill_with_other_block_sizes_in_two_steps(dtype, hq, hkv, d, bs, lengths, cached):
    """A 16-bit cache whose block size is not a multiple of 16: with max_seqlen_k the operator copies the batch's keys
    and values into a temporary cache of 16-token blocks and runs the MFMA kernels over it.  The copy is exact, so the
    result equals the one-step prefill over the same keys in a cache of 16-token blocks bit for bit, and it meets the
    bounds against the oracle; without max_seqlen_k the call runs on the generic kernel (same bounds)."""
    c = make_paged_prefill_case(75, lengths, cached, hq, hkv, d, bs, dtype=dtype)
    scale = 1 / math.sqrt(d)
    args = (c["q_new"].to(DEV), c["k_cache"].to(DEV), c["v_cache"].to(DEV), c["block_tables"].to(DEV), c["cu_q"].to(DEV),
            c["cu_k"].to(DEV), scale, hq, hkv, d, bs)
    got = flash_attention_prefill_paged(*args, max_seqlen_k=max(lengths) + 7).cpu()
    want = _oracle32(c, scale, hq, hkv, d, bs)
    _check(got, want, dtype)
    c16 = make_paged_prefill_case(75, lengths, cached, hq, hkv, d, 16, dtype=dtype)       # same seed: the same q, k, v
    assert torch.equal(c16["q_new"], c["q_new"])
    assert torch.equal(got, _run(c16, scale, hq, hkv, d, 16))
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _check(flash_attention_prefill_paged(*args).cpu(), want, dtype)


@pytest.mark.parametrize("hq,hkv,new,cached", [(16, 8, 4, 846), (10, 1, 5, 1873), (40, 4, 5, 72), (2, 1, 3, 833),
                                               (32, 8, 4, 846), (16, 8, 1, 0), (16, 8, 129, 1)])
def test_two_group_paged_prefill_short_tail_behind_a_long_prefix(hq, hkv, new, cached):
    """One sequence, a few new tokens behind a prefix that ends early in a key tile: an item of 128 rows ranks by the tile
    of its block's last row, up to two tiles past the sequence's last key, and the walk over the ranks has to start
    above it (a walk that started at the last key's tile left such an item to no workgroup).  The output starts as
    NaN."""
    d, bs = 128, 16
    c = make_paged_prefill_case(71, [new + cached], [cached], hq, hkv, d, bs, dtype=torch.float16)
    scale = 1 / math.sqrt(d)
    from minivllm_amd import _C
    q_new = c["q_new"].to(DEV)
    out = torch.full_like(q_new, float("nan"))
    kc, vc, bt, cuq, cuk = (c[k].to(DEV) for k in ("k_cache", "v_cache", "block_tables", "cu_q", "cu_k"))
    st = _C.load().mvllm_prefill_paged(out.data_ptr(), q_new.data_ptr(), kc.data_ptr(), vc.data_ptr(), bt.data_ptr(),
                                       bt.shape[1], cuq.data_ptr(), cuk.data_ptr(), 1, q_new.shape[0], hq, hkv, d, bs,
                                       kc.shape[0], scale, _C.dtype_code(q_new.dtype), _C.current_stream_ptr(out.device))
    torch.cuda.synchronize()
    assert st == 0
    _check(out.cpu(), _oracle32(c, scale, hq, hkv, d, bs), torch.float16)


@pytest.mark.parametrize("hq,hkv,d,bs", [(16, 8, 64, 16), (32, 8, 128, 16), (6, 2, 64, 48)])
def test_int8_paged_prefill_short_sequences(hq, hkv, d, bs):
    """Queries with one to a dozen keys over an INT8 cache (head_dim 64 with two keys is the case a long random run
    once found 0.022 from the oracle).  Nothing averages out there: a row with one key returns that key's dequantised
    value, code * scale in fp32, which a 16-bit output cannot hold exactly; at |value| >= 4 half a bf16 step is 0.0156
    by itself, and the weights' rounding to 16 bits adds up to |value| * 2^-9 more.  Feeding the matrix unit exact
    codes with the scales on the scores and the weights (as INT8 decode does) was tried on 900 such cases: the worst
    difference beyond the output's half step was 0.0149 either way, so the bound below is max-abs 2e-2 beyond that
    half step (fp16 outputs: practically the plain bound) and mean-abs 2e-3, on 40 batches per shape."""
    from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8, store_kvcache_int8
    scale = 1 / math.sqrt(d)
    for seed in range(40):
        g = torch.Generator().manual_seed(5000 + seed)
        nseq = int(torch.randint(2, 9, (1,), generator=g))
        lengths = torch.randint(1, 12, (nseq,), generator=g).tolist()
        if seed == 0:
            lengths[0] = 2                                        # a query with exactly two keys, none of them cached
        cached = [int(torch.randint(0, n, (1,), generator=g)) for n in lengths]
        if seed == 0:
            cached[0] = 0
        dtype = torch.bfloat16 if seed % 2 == 0 else torch.float16
        c = make_paged_prefill_case(seed, lengths, cached, hq, hkv, d, bs, dtype=dtype, poison=0.0)
        nb = c["k_cache"].shape[0]
        ck, cv = (torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV) for _ in range(2))
        sk, sv = (torch.zeros(nb, bs, hkv, device=DEV) for _ in range(2))
        store_kvcache_int8(c["k_cache"].view(-1, hkv, d).to(DEV), c["v_cache"].view(-1, hkv, d).to(DEV), ck, cv, sk, sv,
                           torch.arange(nb * bs, device=DEV), bs)
        got = flash_attention_prefill_paged_int8(c["q_new"].to(DEV), ck, cv, sk, sv, c["block_tables"].to(DEV),
                                                 c["cu_q"].to(DEV), c["cu_k"].to(DEV), scale, hq, hkv, d, bs).cpu()
        kd = oracle.dequantize_cache_oracle(ck.cpu(), sk.cpu())
        vd = oracle.dequantize_cache_oracle(cv.cpu(), sv.cpu())
        want = oracle.prefill_paged_oracle(c["q_new"].float(), kd, vd, c["block_tables"], c["cu_q"], c["cu_k"], scale,
                                           hq, hkv, d, bs)
        mx, mean = error_stats(got, want)
        excess = ((got.float() - want).abs() - half_step(want, dtype)).max().item()
        assert excess <= 2e-2 and mean <= 2e-3, (seed, lengths, cached, str(dtype), mx, excess, mean)


def test_attention_module_batched_4d_prefill_over_cached_prefix():
    """Batched mode of Attention.forward (attention.py:526-533: q (B, N, Hq, D)) with block tables in the context:
    every sequence brings N new tokens after its own cached prefix; the rows are packed with equal cu_seqlens_q and
    run on the paged prefill.  Output (B, N, Hq * D), against the paged-prefill oracle."""
    from minivllm_amd.layers.attention import Attention
    from minivllm_amd.utils import reset_context, set_context
    hq, hkv, d, bs, n = 8, 2, 128, 16, 40
    cached = [32, 0, 96]
    kv_lengths = [c + n for c in cached]
    c = make_paged_prefill_case(71, kv_lengths, cached, hq, hkv, d, bs, dtype=torch.bfloat16)
    layer = Attention(hq, d, 1.0, hkv, bs)
    layer.k_cache, layer.v_cache = c["k_cache"].to(DEV), c["v_cache"].to(DEV)
    k_new, v_new = c["k"][c["new_rows"]].contiguous(), c["v"][c["new_rows"]].contiguous()
    # slot_mapping None: the cache already holds the new tokens' keys (the helper stored every key)
    set_context(True, None, c["cu_k"].to(DEV), n, max(kv_lengths), None, None, c["block_tables"].to(DEV))
    out = layer(c["q_new"].view(3, n, hq, d).to(DEV), k_new.view(3, n, hkv, d).to(DEV), v_new.view(3, n, hkv, d).to(DEV))
    reset_context()
    assert out.shape == (3, n, hq * d)
    want = _oracle32(c, 1 / math.sqrt(d), hq, hkv, d, bs)
    _check(out.cpu().view(3 * n, hq, d), want, torch.bfloat16)
