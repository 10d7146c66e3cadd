"""flash_attention_prefill on the GPU vs the CPU oracle (tolerances as in test_gpu_decode)."""
import math

import pytest
import torch

import oracle
from helpers import error_stats, make_slot_mapping, make_varlen_case
from minivllm_amd.layers.attention import Attention, flash_attention_prefill, paged_attention_decode
from minivllm_amd.utils import reset_context, set_context

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAX_ABS_16, MEAN_ABS_16, MAX_ABS_32 = 2e-2, 2e-3, 2e-4


def _run(q, k, v, cu, scale, hq, hkv, d):
    out = flash_attention_prefill(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), scale, hq, hkv, d)
    torch.cuda.synchronize()
    return out.cpu()


def _oracle32(q, k, v, cu, scale, hq, hkv, d):
    return oracle.prefill_standard_oracle(q.float(), k.float(), v.float(), cu, scale, hq, hkv, d)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,d,lengths", [
    (32, 8, 128, [64, 1, 130, 257, 31]),
    (16, 8, 128, [96, 33, 32, 128]),
    (8, 8, 128, [200]),
    (16, 16, 64, [60, 60]),             # the reference demo's head_dim
    (6, 2, 80, [17, 5]),                # 16-bit: the 16-row tile kernel with a partial last step; fp32: generic
    (6, 2, 72, [17, 5]),                # 16-bit: the 16-row tile kernel, the last step half empty; fp32: generic
    (6, 2, 100, [17, 5]),               # a head_dim no matrix-unit kernel takes
    (6, 2, 128, [300, 17, 64]),         # three query heads per kv head: one head per workgroup
    (10, 2, 128, [33, 129]),            # five
])
def test_prefill_vs_oracle(dtype, hq, hkv, d, lengths):
    case = make_varlen_case(51, lengths, hq, hkv, d, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d)
    want = _oracle32(*case, scale, hq, hkv, d)
    mx, mean = error_stats(got, want)
    assert got.dtype == dtype and got.shape == want.shape
    if dtype == torch.float32:
        assert mx <= MAX_ABS_32, mx
    else:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,lengths", [
    (8, 4, 32, [64, 17, 130]), (8, 2, 96, [70, 1, 33, 129]), (6, 6, 96, [200]), (8, 2, 80, [70, 1, 33, 129]),
    (6, 3, 112, [200, 17]),
    (32, 8, 96, [300, 64, 1, 129, 513]), (16, 2, 112, [1000, 17]), (4, 1, 80, [257, 256, 255]), (16, 16, 32, [90, 700]),
    (8, 2, 256, [70, 1, 33, 129]), (4, 4, 256, [200]), (6, 3, 256, [300, 65, 700]), (4, 4, 48, [200]), (8, 2, 48, [70, 1, 33, 129]),
])
def test_prefill_head_dim_32_80_96_112_256_on_the_lds_tiled_kernel(dtype, hq, hkv, d, lengths):
    """The tiled kernel in the layout of the next larger of 64 / 128 (the reference's kernel takes any head_dim by
    tile table, attention.py:249-257): the chunks of a tile row past the head hold the neighbouring head's data, which
    no product may pick up.  Every head, 4 / 2 / 1 query heads per kv head in a workgroup, ragged ends.  head_dim 256
    is a layout of its own (512-byte tile rows, one workgroup per CU)."""
    from minivllm_amd.layers.attention import prefill_plan
    assert prefill_plan(hq, hkv, d, 0, dtype) == 2
    case = make_varlen_case(55, lengths, hq, hkv, d, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d)
    assert torch.isfinite(got.float()).all()
    mx, mean = error_stats(got, _oracle32(*case, scale, hq, hkv, d))
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d,lengths", [(8, 2, 40, [70, 1, 33, 129]), (8, 4, 56, [64, 17, 130]),
                                              (8, 2, 72, [70, 1, 33, 129]), (6, 3, 88, [200, 17]), (6, 6, 104, [150]),
                                              (8, 2, 120, [70, 1, 33, 129]), (16, 8, 72, [700, 300]), (5, 5, 40, [257, 64]),
                                              (12, 4, 104, [513, 1, 90])])
def test_prefill_head_dims_that_are_multiples_of_8_on_the_lds_tiled_kernel(dtype, hq, hkv, d, lengths):
    """Multiples of 8 that are not multiples of 16: the last 16-dim step of the first product holds 8 dims; its upper
    lanes carry zeros as Q and the row's first chunk as K (what follows the head in memory is the next head, not
    zeros)."""
    from minivllm_amd.layers.attention import prefill_plan
    assert prefill_plan(hq, hkv, d, 0, dtype) == 2
    case = make_varlen_case(57, lengths, hq, hkv, d, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d)
    mx, mean = error_stats(got, _oracle32(*case, scale, hq, hkv, d))
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hkv,d", [(4, 2, 256), (8, 2, 128), (4, 1, 96), (4, 2, 64), (16, 8, 128)])
def test_prefill_running_maximum_moves_in_later_tiles(dtype, hq, hkv, d):
    """Keys whose norm grows with their position (and queries five times the usual size) make the row maxima jump by
    more than the lazy-rescale threshold in tile after tile, so the accumulators that already hold several tiles are
    scaled down again and again (head_dim 256 does this on the accumulator half of the register file directly).
    fp16 meets the usual bounds.  bf16 does not at logits this large, in any kernel and for a reason that has nothing
    to do with the rescaling: the queries enter the matrix unit as q * scale * log2 e rounded to 8 bits of mantissa,
    and an error of 2^-9 of a logit near 40 is 8 % of a weight (measured: 0.06-0.11 max, 0.0021-0.0022 mean for every
    head_dim), so bf16 gets bounds that a lost or doubled rescale (errors of order one) still fails by far."""
    lengths = [700, 130, 333]
    q, k, v, cu = make_varlen_case(57, lengths, hq, hkv, d, dtype=dtype)
    ramp = torch.cat([torch.linspace(0.5, 3.0, n) for n in lengths]).to(k.device)
    q = (q.float() * 5).to(dtype)
    k = (k.float() * ramp[:, None, None]).to(dtype)
    scale = 1 / math.sqrt(d)
    got = _run(q, k, v, cu, scale, hq, hkv, d)
    assert torch.isfinite(got.float()).all()
    mx, mean = error_stats(got, _oracle32(q, k, v, cu, scale, hq, hkv, d))
    if dtype == torch.float16:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    else:
        assert mx <= 0.2 and mean <= 4e-3, (mx, mean)


@pytest.mark.parametrize("d", [96, 72, 40, 120])
def test_prefill_other_head_dims_ignore_what_follows_the_head(d):
    """head_dim 96: the last two chunks of each 256-byte tile row are copied from whatever follows the head in memory
    (72, 40, 120: the same, and the last step of the first product is half empty).
    With the next head (and for the last head the next token) poisoned by huge values and NaNs in one run, the outputs
    of every head must equal those of the clean run bit for bit."""
    hq, hkv = 8, 2
    q, k, v, cu = make_varlen_case(56, [150, 31, 64], hq, hkv, d, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    clean = _run(q, k, v, cu, scale, hq, hkv, d)
    for victim in range(hkv):
        k2, v2 = k.clone(), v.clone()
        other = 1 - victim
        k2[:, other] = float("nan")
        v2[:, other] = float("inf")
        got = _run(q, k2, v2, cu, scale, hq, hkv, d)
        group = hq // hkv
        keep = slice(victim * group, (victim + 1) * group)
        assert torch.equal(got[:, keep], clean[:, keep])


def test_prefill_zero_length_sequences_and_independence():
    hq, hkv, d = 8, 2, 128
    lengths = [0, 70, 0, 0, 129, 0]
    q, k, v, cu = make_varlen_case(52, lengths, hq, hkv, d, dtype=torch.bfloat16)
    got = _run(q, k, v, cu, 0.09, hq, hkv, d)
    want = _oracle32(q, k, v, cu, 0.09, hq, hkv, d)
    assert error_stats(got, want)[0] <= MAX_ABS_16
    # first row of each sequence is exactly its own V row (softmax over one element)
    for start in (0, 70):
        for h in range(hq):
            assert torch.equal(got[start, h], v[start, h // 4])
    # sequences are independent: changing the second prompt leaves the first bit-identical
    k2, v2 = k.clone(), v.clone()
    k2[70:] = 1.0
    v2[70:] = -1.0
    got2 = _run(q, k2, v2, cu, 0.09, hq, hkv, d)
    assert torch.equal(got[:70], got2[:70])


@pytest.mark.parametrize("hq,hkv", [(4, 1), (4, 2), (3, 3)])        # 4, 2 and 1 query heads of a kv head per workgroup
@pytest.mark.parametrize("num_seqs", [64, 65, 130])
def test_prefill_item_order_covers_every_tile(hq, hkv, num_seqs):
    """Up to 64 sequences the workgroups take their (sequence, row tile) from the heaviest-first banded order, beyond
    that from the plain one.  Ragged lengths around the band and tile boundaries (0, 1, 31..33, 255..257, 511..513,
    700) in a shuffled order: every row of every sequence must come out right, so no tile is skipped or doubled."""
    d = 128
    g = torch.Generator().manual_seed(500 + num_seqs)
    pool = [0, 1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 512, 513, 700]
    lengths = [pool[i] for i in torch.randint(0, len(pool), (num_seqs,), generator=g).tolist()]
    lengths[num_seqs // 2] = 700
    lengths[-1] = 257
    q, k, v, cu = make_varlen_case(53, lengths, hq, hkv, d, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    poison = torch.full_like(q, float("nan"))                       # a skipped tile would leave its rows untouched
    from minivllm_amd import _C
    out = poison.to(DEV)
    qd, kd, vd, cud = (t.to(DEV) for t in (q, k, v, cu))
    st = _C.load().mvllm_prefill_varlen(out.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), cud.data_ptr(),
                                        num_seqs, q.shape[0], hq, hkv, d, scale, _C.dtype_code(q.dtype),
                                        _C.current_stream_ptr(out.device))
    torch.cuda.synchronize()
    assert st == 0
    got = out.cpu()
    assert torch.isfinite(got).all()
    want = _oracle32(q, k, v, cu, scale, hq, hkv, d)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("hq,hkv,dtype", [(32, 8, torch.bfloat16), (64, 8, torch.bfloat16), (24, 2, torch.bfloat16),
                                          (8, 2, torch.bfloat16), (12, 3, torch.bfloat16), (4, 1, torch.bfloat16),
                                          (16, 8, torch.bfloat16), (16, 8, torch.float16), (12, 2, torch.bfloat16),
                                          (2, 1, torch.bfloat16), (20, 2, torch.float16)])
@pytest.mark.parametrize("num_seqs", [1, 7, 64])
def test_two_group_prefill_deals_every_item_once(hq, hkv, dtype, num_seqs):
    """The two-group kernel (head_dim 128, an even number of query heads per kv head, at most 64 sequences).  Items of
    four heads and 64 rows: one to three slices of four query heads per kv head, 1 / 2 / 3 / 6 / 8 / 16 slices in
    1 / 2 / 8 teams of workgroups, rounds dealt forwards, backwards and a short last round backwards.  Items of two heads
    and 128 rows (2, 6 or 10 query heads per kv head): 1 / 6 / 8 / 10 slices, the diagonal through an item's last two
    tiles, the waves of the first 64 rows masking all of the last one.  Ragged lengths around the block boundaries,
    empty sequences and one long prompt; the output starts as NaN, so an item that no workgroup took would show, and an
    item taken twice or with the wrong heads would be wrong against the oracle."""
    d = 128
    g = torch.Generator().manual_seed(900 + 7 * num_seqs + hq)
    pool = [0, 1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 257, 300, 448]
    lengths = [pool[i] for i in torch.randint(0, len(pool), (num_seqs,), generator=g).tolist()]
    lengths[num_seqs // 2] = 2100 if hq <= 32 else 700           # 33 (or 11) blocks of 64 rows
    q, k, v, cu = make_varlen_case(58, lengths, hq, hkv, d, dtype=dtype)
    scale = 1 / math.sqrt(d)
    from minivllm_amd import _C
    out = torch.full_like(q, float("nan")).to(DEV)
    qd, kd, vd, cud = (t.to(DEV) for t in (q, k, v, cu))
    st = _C.load().mvllm_prefill_varlen(out.data_ptr(), qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), cud.data_ptr(),
                                        num_seqs, q.shape[0], hq, hkv, d, scale, _C.dtype_code(q.dtype),
                                        _C.current_stream_ptr(out.device))
    torch.cuda.synchronize()
    assert st == 0
    got = out.cpu()
    assert torch.isfinite(got).all()
    want = _oracle32(q, k, v, cu, scale, hq, hkv, d)
    mx, mean = error_stats(got, want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


def test_config2_full_size():
    """BASELINE.json config 2: 16 prompts L U[64,2048], Hq32/Hkv8/D128 bf16; store into block-256 cache; the last
    row of each prompt must agree with a paged decode of that token over the stored cache."""
    hq, hkv, d, bs = 32, 8, 128, 256
    g = torch.Generator().manual_seed(53)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    q, k, v, cu = make_varlen_case(54, lengths, hq, hkv, d, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    slots, tables, nb = make_slot_mapping(55, lengths, bs)
    layer = Attention(hq, d, 1.0, hkv, bs)
    layer.k_cache = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=DEV)
    layer.v_cache = torch.zeros_like(layer.k_cache)
    set_context(True, cu.to(DEV), cu.to(DEV), max(lengths), max(lengths), slots.to(DEV), None, None)
    out = layer(q.to(DEV), k.to(DEV), v.to(DEV))
    reset_context()
    assert out.shape == (sum(lengths), hq * d)
    out = out.cpu().view(-1, hq, d)
    # oracle on the three shortest and the longest prompt (O(L^2) on CPU)
    order = sorted(range(16), key=lambda i: lengths[i])
    for s in order[:3] + order[-1:]:
        lo, hi = int(cu[s]), int(cu[s + 1])
        sub_cu = torch.tensor([0, hi - lo], dtype=torch.int32)
        want = _oracle32(q[lo:hi], k[lo:hi], v[lo:hi], sub_cu, scale, hq, hkv, d)
        mx, mean = error_stats(out[lo:hi], want)
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (s, hi - lo, mx, mean)
    # size-independent cross-check over all prompts: last prefill row == decode over the stored cache
    width = max(len(t) for t in tables)
    bt = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
    last = (cu[1:] - 1).long()
    dec = paged_attention_decode(q[last].to(DEV), layer.k_cache, layer.v_cache, bt,
                                 torch.tensor(lengths, device=DEV), scale, hq, hkv, d, bs).cpu()
    mx, mean = error_stats(dec, out[last])
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,lengths", [
    (16, 8, [64, 1, 130, 257, 31]),          # the reference demo's heads (main.py: 16 q / 8 kv heads of 64 dims)
    (12, 12, [200, 15, 16, 17]),             # qwen3.py:333-339 self-test: 12 heads
    (12, 1, [96, 33, 1000]),                 # one kv head
    (6, 2, [17, 0, 5, 0, 48]),               # heads not a multiple of the four waves; empty sequences
])
def test_prefill_head_dim_64_vs_oracle(dtype, hq, hkv, lengths):
    """head_dim 64 runs on the LDS-tiled kernels, 16-bit and fp32 (not on the generic kernel)."""
    d = 64
    case = make_varlen_case(56, lengths, hq, hkv, d, dtype=dtype)
    scale = 1 / math.sqrt(d)
    got = _run(*case, scale, hq, hkv, d)
    want = _oracle32(*case, scale, hq, hkv, d)
    mx, mean = error_stats(got, want)
    assert got.dtype == dtype and got.shape == want.shape
    if dtype == torch.float32:                # main.py's default dtype: the fp32 matrix instructions
        assert mx <= MAX_ABS_32, mx
    else:
        assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    # first row of each sequence is exactly its own V row; rows do not depend on later sequences
    q, k, v, cu = case
    for s, n in enumerate(lengths):
        if n:
            lo = int(cu[s])
            assert torch.equal(got[lo], v[lo].repeat_interleave(hq // hkv, dim=0))
    k2, v2 = k.clone(), v.clone()
    first = next(i for i, n in enumerate(lengths) if n)
    cut = int(cu[first + 1])
    k2[cut:] = 1.0
    v2[cut:] = -1.0
    assert torch.equal(_run(q, k2, v2, cu, scale, hq, hkv, d)[:cut], got[:cut])


def test_attention_module_batched_4d_prefill():
    """Batched mode of Attention.forward (attention.py:526-533: q (B, N, Hq, D); the reference calls a function it
    never defines): B sequences of N tokens, causal inside each, output (B, N, Hq * D); K/V rows are stored to
    their slots on the way, as in the packed mode."""
    from minivllm_amd.layers.attention import Attention
    from minivllm_amd.utils import reset_context, set_context
    hq, hkv, d, bs, bsz, n = 8, 2, 128, 16, 3, 70
    q, k, v, cu = make_varlen_case(54, [n] * bsz, hq, hkv, d, dtype=torch.bfloat16)
    layer = Attention(hq, d, 1.0, hkv, bs)
    nb = bsz * (-(-n // bs))
    layer.k_cache = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=DEV)
    layer.v_cache = torch.zeros_like(layer.k_cache)
    slots = torch.cat([torch.arange(n) + s * (-(-n // bs)) * bs for s in range(bsz)])
    set_context(True, None, None, n, n, slots.to(DEV), None, None)          # no cu_seqlens: the shape carries it
    out = layer(q.view(bsz, n, hq, d).to(DEV), k.view(bsz, n, hkv, d).to(DEV), v.view(bsz, n, hkv, d).to(DEV))
    reset_context()
    assert out.shape == (bsz, n, hq * d)
    want = _oracle32(q, k, v, cu, 1 / math.sqrt(d), hq, hkv, d)
    mx, mean = error_stats(out.cpu().view(bsz * n, hq, d), want)
    assert mx <= MAX_ABS_16 and mean <= MEAN_ABS_16, (mx, mean)
    assert torch.equal(layer.k_cache.view(-1, hkv, d)[slots.to(DEV)].cpu(), k)
