"""add_rms_norm and silu_and_mul on the GPU vs the CPU oracle of the reference's tensor-operation chains.

Tolerances.  add_rms_norm: the residual sum is bit-exact; the norm differs from the oracle only through the
order of the sum of squares, so for bf16/fp16 at least 99.5 % of the elements are bit-exact and all are within
1 ulp (2^-7 / 2^-10 relative), fp32 within 2^-19 relative (a sum of up to 8192 squares in another order).  silu_and_mul: exp differs from the CPU's by an ulp or
two of fp32, which the rounding to bf16/fp16 absorbs except at rounding boundaries: same bars, with 2 ulp for
the product (a silu that rounds the other way moves it by one more)."""
import pytest
import torch

import oracle
from minivllm_amd.layers.fused import add_rms_norm, silu_and_mul

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ULP = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -19}


def _close(got, want, dtype, ulps=1.0):
    got = got.cpu()
    assert got.dtype == dtype and got.shape == want.shape
    if dtype != torch.float32:
        same = (got == want).float().mean().item()
        assert same >= 0.995, f"only {same:.4f} bit-exact"
    err = (got.float() - want.float()).abs()
    assert bool((err <= want.float().abs() * ULP[dtype] * ulps + 1e-30).all()), float(err.max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,hidden", [(64, 1024), (1, 1024), (7, 4096), (3, 8), (5, 520), (2, 8192), (300, 2048)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_add_rms_norm(dtype, rows, hidden, with_residual):
    g = torch.Generator().manual_seed(rows * 31 + hidden)
    x = (torch.randn(rows, hidden, generator=g) * 2).to(dtype)
    r = torch.randn(rows, hidden, generator=g).to(dtype) if with_residual else None
    gamma = torch.rand(hidden, generator=g) + 0.5
    if with_residual:
        want_y, want_s = oracle.add_rms_norm_oracle(x, gamma, 1e-6, r)
        got_y, got_s = add_rms_norm(x.to(DEV), gamma.to(DEV), 1e-6, r.to(DEV))
        assert torch.equal(got_s.cpu().view(torch.uint8), want_s.view(torch.uint8))
    else:
        want_y = oracle.add_rms_norm_oracle(x, gamma, 1e-6)
        got_y = add_rms_norm(x.to(DEV), gamma.to(DEV), 1e-6)
    _close(got_y, want_y, dtype)


def test_add_rms_norm_strided_rows_and_errors():
    g = torch.Generator().manual_seed(2)
    wide = torch.randn(9, 3 * 512, generator=g).to(torch.bfloat16)
    gamma = torch.ones(512)
    x = wide.to(DEV)[:, 512:1024]                                  # row stride 1536
    got = add_rms_norm(x, gamma.to(DEV), 1e-5)
    _close(got, oracle.add_rms_norm_oracle(wide[:, 512:1024], gamma, 1e-5), torch.bfloat16)
    with pytest.raises(ValueError):
        add_rms_norm(x, gamma.to(DEV)[:100], 1e-5)
    with pytest.raises(ValueError):
        add_rms_norm(torch.zeros(2, 12, device=DEV), torch.ones(12, device=DEV), 1e-5)      # hidden % 8
    assert add_rms_norm(torch.zeros(0, 64, device=DEV), torch.ones(64, device=DEV), 1e-5).shape == (0, 64)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,width", [(64, 3072), (1, 8), (33, 1000), (1000, 512)])
def test_silu_and_mul(dtype, rows, width):
    g = torch.Generator().manual_seed(rows + width)
    x = (torch.randn(rows, 2 * width, generator=g) * 3).to(dtype)
    want = oracle.silu_and_mul_oracle(x)
    got = silu_and_mul(x.to(DEV))
    _close(got, want, dtype, ulps=2.0)      # one ulp of the rounded silu moves the product by up to one more
    # strided input rows (a slice of a wider buffer)
    wide = torch.zeros(rows, 2 * width + 64, dtype=dtype)
    wide[:, : 2 * width] = x
    _close(silu_and_mul(wide.to(DEV)[:, : 2 * width]), want, dtype, ulps=2.0)
