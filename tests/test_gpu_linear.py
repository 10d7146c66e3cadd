"""linear_small_m (the decode step's projections as one HIP launch) against the fp32 product of the same 16-bit
inputs.  Tolerance: the result is the fp32 sum rounded once to the element type, so |err| <= 2^-8 |want| (bf16; 2^-11
for fp16) plus fp32 summation-order noise, allowed as 2e-3 absolute."""
import pytest
import torch
import torch.nn.functional as F

from minivllm_amd.layers.basic import Linear
from minivllm_amd.layers.fused import (add_rms_norm, decode_advance, linear_small_m, linear_small_m_takes,
                                       norm_linear_small_m, norm_linear_small_m_takes, silu_and_mul)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, m, n, k, dtype, bias, stride=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, stride or k, generator=g).to(dtype).to(DEV)[:, :k]
    w = (torch.randn(n, k, generator=g) * 0.05).to(dtype).to(DEV)
    b = (torch.randn(n, generator=g) * 0.5).to(dtype).to(DEV) if bias else None
    return x, w, b


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m", [1, 3, 16, 17, 33, 48, 60, 64])
@pytest.mark.parametrize("n,k,bias", [(4096, 1024, False), (1024, 2048, False), (6144, 1024, True), (1024, 3072, True),
                                      (48, 512, True), (16, 8192, False)])
def test_linear_small_m_vs_fp32_product(dtype, m, n, k, bias):
    """The engine's four projection shapes (QKV, output, gate/up, down) and the extremes of the wave split: few
    columns with a long K (16 waves share a column tile) and a short K."""
    x, w, b = _case(70 + m, m, n, k, dtype, bias)
    assert linear_small_m_takes(x, w)
    got = linear_small_m(x, w, b).float().cpu()
    want = (x.float() @ w.float().T + (b.float() if bias else 0)).cpu()
    assert got.shape == (m, n)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    slack = ((got - want).abs() - want.abs() * ulp).max().item()
    assert slack <= 2e-3, slack


def test_linear_small_m_strided_rows_and_module_dispatch():
    """Rows of x may be slices of a wider tensor; the module takes the HIP launch up to its row limit and the
    library GEMM beyond, with the same result up to the rounding of the output."""
    x, w, b = _case(90, 24, 1024, 1024, torch.bfloat16, True, stride=1536)
    assert x.stride(0) == 1536 and linear_small_m_takes(x, w)
    want = F.linear(x, w, b).float()
    got = linear_small_m(x, w, b).float()
    assert (got - want).abs().max().item() <= 0.05 and (got - want).abs().mean().item() <= 2e-3
    lin = Linear(1024, 1024, bias=True, small_rows=32).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
        small = lin(x.contiguous())
        big = lin(x.contiguous().repeat(4, 1))                    # 96 rows: F.linear
    assert big.shape == (96, 1024)
    assert (small.float() - big[:24].float()).abs().max().item() <= 0.05
    assert torch.equal(small, linear_small_m(x.contiguous(), w, b))
    assert not linear_small_m_takes(x.float(), w.float())         # fp32 stays with the library
    assert not linear_small_m_takes(torch.zeros(65, 1024, dtype=torch.bfloat16, device=DEV), w)
    assert not linear_small_m_takes(torch.zeros(40, 1024, dtype=torch.bfloat16, device=DEV), w, max_rows=32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m", [1, 5, 16, 17, 32, 48, 64])
@pytest.mark.parametrize("n,k,bias,glu", [(4096, 1024, False, False), (6144, 1024, True, True), (1024, 2048, True, False),
                                          (2048, 512, True, True), (4096, 1024, True, True)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_norm_linear_equals_the_separate_launches(dtype, m, n, k, bias, glu, with_residual):
    """The fused projection against the launches it replaces (add_rms_norm -> linear_small_m -> silu_and_mul): the
    next residual is bit-identical.  The product may differ only through the sum of squares, added in another order:
    where its last bit differs, a normalised value can round the other way (about one in 2^13 fp16 values, 2^16 in
    bf16), and that one input moves every output of its row by a fraction of a unit in the last place, so a row is
    either bit-identical or has some outputs one unit off: every output within 2 units in the last place of the
    largest output of its row (4 behind the activation), and at least 70 % of all outputs bit-identical."""
    x, w, b = _case(300 + m, m, n, k, dtype, bias)
    x = x.contiguous()
    g = torch.Generator().manual_seed(m)
    gamma = (1 + 0.2 * torch.randn(k, generator=g)).to(DEV)
    res = torch.randn(m, k, generator=g).to(dtype).to(DEV) if with_residual else None
    assert norm_linear_small_m_takes(x, w, 64, glu=glu)   # 17 rows and more: one workgroup per 16 rows and column tile
    normed = add_rms_norm(x, gamma, 1e-6, res)
    normed, want_res = normed if with_residual else (normed, x)
    want = linear_small_m(normed, w, b)
    if glu:
        want = silu_and_mul(want)
    got = norm_linear_small_m(x, w, b, gamma, 1e-6, res, want_residual=with_residual, glu=glu)
    if with_residual:
        got, got_res = got
        assert torch.equal(got_res, want_res)
    assert got.shape == want.shape == (m, n // 2 if glu else n)
    same = (got == want).float().mean().item()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    worst = ((got.float() - want.float()).abs() / want.float().abs().amax(dim=1, keepdim=True)).max().item()
    # with the activation behind it, one unit in the gate and one in the up projection meet in a product: 4 units
    assert same >= 0.7 and worst <= (4 if glu else 2) * ulp, (same, worst)


def test_norm_linear_without_norm_is_the_plain_product_and_glu_pairs_the_right_columns():
    """gamma None: no norm, so the result equals linear_small_m bit for bit, and with glu equals silu_and_mul of it;
    a weight whose gate rows are zero except one column pins the pairing of gate column j with up column j."""
    x, w, b = _case(411, 9, 2048, 1024, torch.bfloat16, True)
    x = x.contiguous()
    assert torch.equal(norm_linear_small_m(x, w, b), linear_small_m(x, w, b))
    assert torch.equal(norm_linear_small_m(x, w, b, glu=True), silu_and_mul(linear_small_m(x, w, b)))
    for m, n, k in ((60, 6144, 1024), (33, 2048, 1024), (64, 96, 512)):     # a workgroup per 16 rows (the engine's MLP at 33-64 rows)
        xm, wm, bm = _case(412 + m, m, n, k, torch.bfloat16, True)
        xm = xm.contiguous()
        assert torch.equal(norm_linear_small_m(xm, wm, bm), linear_small_m(xm, wm, bm))
        assert torch.equal(norm_linear_small_m(xm, wm, bm, glu=True), silu_and_mul(linear_small_m(xm, wm, bm)))
    w2 = torch.zeros_like(w)
    b2 = torch.zeros_like(b)
    j = 437                                              # silu(gate_j) * up_j: only column j can be non-zero
    w2[j] = w[j]
    w2[1024 + j] = w[1024 + j]
    w2[1024 + j + 1] = w[1024 + j + 1]                   # an up column whose gate is zero: silu(0) * up = 0
    out = norm_linear_small_m(x, w2, b2, glu=True).float()
    full = x.float() @ w2.float().T
    gate, up = full[:, j].bfloat16().float(), full[:, 1024 + j].bfloat16().float()
    want = (torch.nn.functional.silu(gate).bfloat16().float() * up).bfloat16().float()
    assert out[:, j].abs().max().item() > 0
    assert (out[:, j] - want).abs().max().item() <= 2.0 ** -7 * want.abs().max().item()
    out[:, j] = 0
    assert out.abs().max().item() == 0


def test_decode_advance_moves_the_step_metadata_forward():
    ids = torch.tensor([5, 6, 7, 8], device=DEV)
    ctx = torch.tensor([10, 256, 3, 0], device=DEV)
    pos = torch.zeros(4, dtype=torch.int64, device=DEV)
    slots = torch.tensor([9, 511, 40, -1], device=DEV)
    sampled = torch.tensor([100, 200, 300], device=DEV)           # a batch of three inside buffers of four
    decode_advance(ids, ctx, pos, slots, sampled)
    torch.cuda.synchronize()
    assert ids.tolist() == [100, 200, 300, 8] and ctx.tolist() == [11, 257, 4, 0]
    assert pos.tolist() == [10, 256, 3, 0] and slots.tolist() == [10, 512, 41, -1]
    # all four rows of a captured batch size: the padding row (context 0, slot -1) stays, and the call counter moves
    step = torch.tensor([41], device=DEV)
    decode_advance(ids, ctx, pos, slots, torch.tensor([1, 2, 3, 4], device=DEV), step=step)
    torch.cuda.synchronize()
    assert ids.tolist() == [1, 2, 3, 8] and ctx.tolist() == [12, 258, 5, 0] and slots.tolist() == [11, 513, 42, -1]
    assert pos.tolist() == [11, 257, 4, 0] and step.item() == 42
    # the ids also go to pinned host memory: the row is the counter's parity before the increment, its last entry the
    # new counter value, written after the ids (the host may read the ids once it sees it)
    host = torch.zeros(2, 6, dtype=torch.int64, pin_memory=True)
    decode_advance(ids, ctx, pos, slots, torch.tensor([9, 8, 7, 6], device=DEV), step=step, host_ids=host)   # 42: row 0
    decode_advance(ids, ctx, pos, slots, torch.tensor([5, 4, 3, 2], device=DEV), step=step, host_ids=host)   # 43: row 1
    torch.cuda.synchronize()
    assert host[0].tolist() == [9, 8, 7, 6, 0, 43] and host[1].tolist() == [5, 4, 3, 2, 0, 44] and step.item() == 44
    with pytest.raises(ValueError):
        decode_advance(ids, ctx, pos, slots, sampled, step=step, host_ids=torch.zeros(2, 6, dtype=torch.int64))   # not pinned
    with pytest.raises(ValueError):
        decode_advance(ids, ctx, pos, slots, sampled, host_ids=host)                                             # no counter
