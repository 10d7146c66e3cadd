"""paged_attention_decode on the GPU vs the CPU oracle.

Tolerances (BASELINE.json north_star): bf16/fp16 outputs max-abs <= 2e-2 and
mean-abs <= 2e-3 against the oracle evaluated in fp32 on the same (upcast)
inputs; fp32 outputs max-abs <= 2e-4."""
import math

import pytest
import torch

import oracle
from helpers import error_stats, extract_sequence, make_paged_case, make_paged_case_on_device
from minivllm_amd.layers.attention import Attention, paged_attention_decode, paged_decode_plan
from minivllm_amd.utils import reset_context, set_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16, MAX_ABS_32 = 2e-2, 2e-3, 2e-4


def _run(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs, ctx_dtype=torch.int32):
    out = paged_attention_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), tables.to(DEV), ctx.to(ctx_dtype).to(DEV),
                                 scale, hq, hkv, d, bs)
    torch.cuda.synchronize()
    return out.cpu()


def _oracle32(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs):
    return oracle.decode_naive_oracle(q.float(), kc.float(), vc.float(), tables, ctx, scale, hq, hkv, d, bs)


def test_config1_fp32_elementwise():
    """BASELINE.json config 1: B 8, ctx U[16,512], Hq16/Hkv8, D128, bs16, fp32 cache, shuffled tables."""
    hq, hkv, d, bs = 16, 8, 128, 16
    case = make_paged_case(31, 8, 16, 512, hq, hkv, d, bs)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d, bs)
    want = oracle.decode_naive_oracle(*case, scale, hq, hkv, d, bs)
    want2 = oracle.decode_vectorised_oracle(*case, scale, hq, hkv, d, bs)
    assert got.dtype == torch.float32 and got.shape == want.shape
    assert error_stats(got, want)[0] <= MAX_ABS_32 and error_stats(got, want2)[0] <= MAX_ABS_32


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,bs,ctx_hi", [
    (32, 8, 16, 700),      # GQA 4, multi-partition
    (32, 8, 256, 1500),    # big blocks
    (16, 8, 16, 255),      # GQA 2, single partition (direct output)
    (8, 8, 32, 300),       # MHA
    (32, 4, 16, 600),      # GQA 8
    (6, 2, 48, 500),       # GQA 3, block size not a power of two
    (16, 1, 16, 900),      # MQA with 16 heads: every column of the score product is a live head
    (24, 2, 32, 400),      # GQA 12: live heads in three of the four accumulator row groups
    (5, 1, 16, 300),       # GQA 5: live heads end inside a row group
])
def test_fast_path_vs_oracle(dtype, hq, hkv, bs, ctx_hi):
    d = 128
    case = make_paged_case(32, 9, 1, ctx_hi, hq, hkv, d, bs, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d, bs, ctx_dtype=torch.int64)
    want = _oracle32(*case, scale, hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    assert got.dtype == dtype and mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("bs", [16, 8, 1])
@pytest.mark.parametrize("ctx_list", [[1, 2, 15, 16, 17], [255, 256, 257, 511, 512, 513], [31, 32, 33, 1024, 1025]])
def test_context_length_boundaries(ctx_list, bs):
    hq, hkv, d = 8, 2, 128
    case = make_paged_case(33, 0, 0, 0, hq, hkv, d, bs, dtype=torch.bfloat16, ctx_list=ctx_list)
    got = _run(*case, 0.1, hq, hkv, d, bs)
    want = _oracle32(*case, 0.1, hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype,hq,hkv,d,bs", [
    (torch.float32, 4, 2, 64, 4),       # generic kernel: fp32 with a block size of 4
    (torch.float32, 6, 2, 96, 16),      # fp32, head_dim 96
    (torch.bfloat16, 16, 16, 64, 8),    # head_dim 64, blocks of 8 tokens (the MFMA kernel's small-block form)
    (torch.bfloat16, 4, 2, 128, 12),    # a block size that neither divides 16 nor is a multiple of it
    (torch.float32, 16, 8, 64, 16),     # the reference demo's shape and dtype (main.py)
    (torch.float16, 6, 3, 80, 3),       # odd head_dim and block size
    (torch.bfloat16, 4, 1, 256, 16),
])
def test_generic_path_vs_oracle(dtype, hq, hkv, d, bs):
    case = make_paged_case(34, 5, 1, 400, hq, hkv, d, bs, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d, bs)
    want = _oracle32(*case, scale, hq, hkv, d, bs)
    mx, mean = error_stats(got, want)
    if dtype == torch.float32:
        assert mx <= MAX_ABS_32, mx
    else:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


def test_padded_rows_zero_context_and_missing_blocks():
    """Graph-replay padding (context_len 0, stale table rows) gives zero rows; tokens whose table entry is -1
    contribute nothing (attention.py:350-355)."""
    hq, hkv, d, bs = 8, 2, 128, 16
    q, kc, vc, tables, ctx = make_paged_case(35, 0, 0, 0, hq, hkv, d, bs, dtype=torch.bfloat16,
                                             ctx_list=[40, 0, 300, 64])
    tables[1] = 0                       # stale entries on the padded row
    got = _run(q, kc, vc, tables, ctx, 0.09, hq, hkv, d, bs)
    assert torch.count_nonzero(got[1]) == 0 and torch.isfinite(got).all()
    keep = [0, 2, 3]
    want = _oracle32(q[keep], kc, vc, tables[keep], ctx[keep], 0.09, hq, hkv, d, bs)
    assert error_stats(got[keep], want)[0] <= MAX_ABS_16
    # knock out the 2nd block of sequence 2 (tokens 16..31): same as attending to the other tokens only
    hole = tables.clone()
    hole[2, 1] = -1
    got2 = _run(q, kc, vc, hole, ctx, 0.09, hq, hkv, d, bs)
    kf, vf = kc.float(), vc.float()
    rows_k = oracle.gather_sequence_kv(kf, tables[2], 300, bs)
    rows_v = oracle.gather_sequence_kv(vf, tables[2], 300, bs)
    sel = torch.cat([torch.arange(0, 16), torch.arange(32, 300)])
    for h in range(hq):
        s = (rows_k[sel, h // 4] @ q[2, h].float()) * 0.09
        want_h = torch.softmax(s, 0) @ rows_v[sel, h // 4]
        assert (got2[2, h].float() - want_h).abs().max() <= MAX_ABS_16
    # a sequence whose every block is missing: zeros
    hole[0, :] = -1
    got3 = _run(q, kc, vc, hole, ctx, 0.09, hq, hkv, d, bs)
    assert torch.count_nonzero(got3[0]) == 0


def test_block_permutation_and_batch_order_invariance():
    hq, hkv, d, bs = 32, 8, 128, 16
    q, kc, vc, tables, ctx = make_paged_case(36, 12, 1, 900, hq, hkv, d, bs, dtype=torch.bfloat16)
    a = _run(q, kc, vc, tables, ctx, 0.088, hq, hkv, d, bs)
    perm = torch.randperm(kc.shape[0], generator=torch.Generator().manual_seed(37))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    t2 = torch.where(tables >= 0, inv[tables.clamp(min=0).long()].to(torch.int32), tables)
    b = _run(q, kc[perm], vc[perm], t2, ctx, 0.088, hq, hkv, d, bs)
    assert torch.equal(a, b)
    order = torch.randperm(12, generator=torch.Generator().manual_seed(38))
    c = _run(q[order], kc, vc, tables[order], ctx[order], 0.088, hq, hkv, d, bs)
    assert torch.equal(a[order], c)


def test_wider_table_same_result():
    """Split-K invariance: a wider (more -1 padded) block table changes the partitioning, not the result."""
    hq, hkv, d, bs = 32, 8, 128, 16
    q, kc, vc, tables, ctx = make_paged_case(39, 6, 1, 1000, hq, hkv, d, bs, dtype=torch.bfloat16)
    a = _run(q, kc, vc, tables, ctx, 0.088, hq, hkv, d, bs)
    wide = torch.full((6, 2048), -1, dtype=torch.int32)
    wide[:, :tables.shape[1]] = tables
    b = _run(q, kc, vc, wide, ctx, 0.088, hq, hkv, d, bs)
    want = _oracle32(q, kc, vc, tables, ctx, 0.088, hq, hkv, d, bs)
    assert error_stats(a, want)[0] <= MAX_ABS_16 and error_stats(b, want)[0] <= MAX_ABS_16
    assert (a.float() - b.float()).abs().max() <= 4e-3


@pytest.mark.parametrize("bs", [16, 256])
def test_config3_full_size_subset_vs_oracle(bs):
    """BASELINE.json config 3: B 256, ctx log-uniform [128, 32768], Hq32/Hkv8/D128 bf16.  The oracle is evaluated on
    a seeded subset of sequences (the padded formulation does not fit in host memory for all 256)."""
    hq, hkv, d = 32, 8, 128
    q, kd, vd, tables, ctx = make_paged_case_on_device(40, DEV, 256, 128, 32768, hq, hkv, d, bs)
    scale = 1 / math.sqrt(d)
    td, cd = tables.to(DEV), ctx.to(DEV)
    got = paged_attention_decode(q, kd, vd, td, cd, scale, hq, hkv, d, bs).cpu()
    assert torch.isfinite(got).all()
    pick = [0, 1, 2, int(ctx.argmax()), int(ctx.argmin()), 100, 200, 255]
    for b in pick:
        kc, vc, table, c = extract_sequence(kd, vd, tables, ctx, b, bs)
        want = _oracle32(q[b:b + 1].cpu(), kc, vc, table, c, scale, hq, hkv, d, bs)
        mx, mean = error_stats(got[b:b + 1], want)
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (b, int(ctx[b]), mx, mean)
    # size-independent property at full size: linearity in V (attention weights do not depend on V)
    vd *= 2
    got2 = paged_attention_decode(q, kd, vd, td, cd, scale, hq, hkv, d, bs).cpu()
    assert (got2.float() - 2 * got.float()).abs().max() <= 2e-2


def test_attention_module_decode_dispatch():
    hq, hkv, d, bs = 16, 8, 128, 256
    q, kc, vc, tables, ctx = make_paged_case(41, 5, 1, 352, hq, hkv, d, bs, dtype=torch.bfloat16)
    layer = Attention(hq, d, 1.0, hkv, bs)
    layer.k_cache, layer.v_cache = kc.to(DEV), vc.to(DEV)
    # the new token's K/V is stored first, then decode reads context_len tokens including it
    g = torch.Generator().manual_seed(42)
    k_new = torch.randn(5, hkv, d, generator=g).to(torch.bfloat16)
    v_new = torch.randn(5, hkv, d, generator=g).to(torch.bfloat16)
    slots = torch.tensor([int(tables[b, (int(ctx[b]) - 1) // bs]) * bs + (int(ctx[b]) - 1) % bs for b in range(5)])
    set_context(False, slot_mapping=slots.to(DEV), context_lens=ctx.to(DEV), block_tables=tables.to(DEV))
    out = layer(q.to(DEV), k_new.to(DEV), v_new.to(DEV))
    reset_context()
    kc2, vc2 = kc.clone(), vc.clone()
    oracle.store_kvcache_oracle(k_new, v_new, kc2, vc2, slots, bs)
    want = _oracle32(q, kc2, vc2, tables, ctx, 1 / math.sqrt(d), hq, hkv, d, bs).reshape(5, hq * d)
    assert out.shape == (5, hq * d)
    mx, mean = error_stats(out.cpu(), want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16


def _pad_tables(tables, width_tokens, bs):
    width = max(tables.shape[1], width_tokens // bs)
    out = torch.full((tables.shape[0], width), -1, dtype=torch.int32)
    out[:, :tables.shape[1]] = tables
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,bs,d", [(32, 8, 16, 128), (16, 8, 256, 128), (16, 1, 32, 128), (24, 2, 16, 128),
                                         (5, 1, 64, 128), (8, 8, 48, 128),
                                         (16, 8, 16, 64), (16, 16, 256, 64), (12, 1, 32, 64), (5, 5, 48, 64),
                                         (34, 2, 16, 128), (48, 1, 32, 128), (71, 1, 16, 64),
                                         (32, 8, 8, 128), (16, 8, 1, 128), (16, 16, 4, 64), (5, 1, 2, 128)])
@pytest.mark.parametrize("form", ["one wave per head", "waves share a head", "waves share a head, one partition"])
def test_both_grid_forms_vs_oracle(dtype, hq, hkv, bs, d, form):
    """A ragged batch (contexts 1..1300, one empty) through both forms of the MFMA kernel: the batch size and the
    width of the block table, not the contexts, decide the form.  64 sequences in a table of 32 K tokens take the
    one-wave-per-head grid; 7 sequences in a table of 8 K tokens are spread over four waves per head in several
    partitions; 64 sequences x 8 kv heads in a table of 4 K tokens are one partition each, written without the
    merge kernel.  head_dim 64 (the reference demo's model, qwen3.py:338) runs on the same kernels with half of
    the second product's columns switched off.  More than 16 query heads per kv head (17, 48, 71) are served in slices
    of 16, the last one partial.  Blocks of 8, 4, 2 and 1 tokens: every lane looks up the blocks of its own tokens."""
    batch = 7 if form == "waves share a head" else 64
    width = {"one wave per head": 32768, "waves share a head": 8192}.get(form, 4096) // bs * bs
    g = torch.Generator().manual_seed(77)
    ctx_list = torch.randint(1, 1301, (batch,), generator=g).tolist()
    ctx_list[3] = 0
    ctx_list[5] = 1300
    q, kc, vc, tables, ctx = make_paged_case(78, 0, 0, 0, hq, hkv, d, bs, dtype=dtype, ctx_list=ctx_list)
    tables = _pad_tables(tables, width, bs)
    assert tables.shape[1] == width // bs
    part, parts, waves = paged_decode_plan(batch, hq, hkv, d, tables.shape[1], bs, dtype)
    if form == "one wave per head":
        assert waves == 1 and part >= 1024
    elif form == "waves share a head":
        assert waves > 1 and parts > 1
    else:
        assert waves > 1 and (parts == 1 or hkv < 8)
    scale = 1 / math.sqrt(d)
    got = _run(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
    live = ctx > 0                                    # the oracle, like the reference, has no answer for an empty context
    want = _oracle32(q[live], kc, vc, tables[live][:, :-(-1300 // bs)], ctx[live], scale, hq, hkv, d, bs)
    mx, mean = error_stats(got[live], want)
    if dtype == torch.float32:                        # fp32 caches: the same kernels on the fp32 matrix instructions
        assert mx <= MAX_ABS_32, mx
    else:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    assert torch.count_nonzero(got[3]) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,bs,d", [(16, 8, 16, 256), (8, 1, 32, 256), (5, 5, 48, 256), (16, 8, 16, 32), (12, 2, 256, 32),
                                         (32, 8, 16, 96), (6, 6, 48, 96), (12, 1, 256, 96), (32, 8, 16, 80), (5, 5, 48, 112),
                                         (12, 1, 256, 80), (16, 2, 32, 112), (16, 8, 16, 72), (6, 2, 32, 88), (8, 8, 16, 40),
                                         (12, 3, 48, 104), (16, 4, 16, 120), (8, 2, 16, 48), (10, 2, 16, 56)])
@pytest.mark.parametrize("form", ["one wave per head", "waves share a head", "waves share a head, one partition"])
def test_head_dim_256_96_and_32_on_the_mfma_kernels(dtype, hq, hkv, bs, d, form):
    """The other head dims the reference's kernels take (attention.py:249-257, 453) that are a multiple of 32: with 256
    dims a lane owns two sets of eight output dims and the first product has eight 32-dim steps; with 96 there are three
    steps and twelve of the sixteen output columns, with 80 and 112 the last step is partial (the lanes past the row's
    end load nothing), with 32 one step and four columns; every other multiple of 8 between 32 and 128 likewise.  Both
    kernel forms, ragged contexts, one empty."""
    batch = 7 if form == "waves share a head" else 64
    width = {"one wave per head": 32768, "waves share a head": 8192}.get(form, 4096) // bs * bs
    g = torch.Generator().manual_seed(177)
    ctx_list = torch.randint(1, 901, (batch,), generator=g).tolist()
    ctx_list[3] = 0
    ctx_list[5] = 900
    q, kc, vc, tables, ctx = make_paged_case(178, 0, 0, 0, hq, hkv, d, bs, dtype=dtype, ctx_list=ctx_list)
    tables = _pad_tables(tables, width, bs)
    part, parts, waves = paged_decode_plan(batch, hq, hkv, d, tables.shape[1], bs, dtype)
    assert waves == (1 if form == "one wave per head" else 4), (part, parts, waves)
    scale = 1 / math.sqrt(d)
    got = _run(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
    live = ctx > 0
    want = _oracle32(q[live], kc, vc, tables[live][:, :-(-900 // bs)], ctx[live], scale, hq, hkv, d, bs)
    mx, mean = error_stats(got[live], want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    assert torch.count_nonzero(got[3]) == 0
