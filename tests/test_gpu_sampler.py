"""sample_tokens on the GPU vs the CPU oracle of the reference's sampler (softmax(logits/T) / noise -> argmax).

The result is an index, so the bar is exact agreement.  The kernel takes the argmax of
logit/T - log(noise) instead of dividing probabilities; the two orders can only differ where two candidates tie
to within float rounding, which random inputs do not produce (and the tests would show as a mismatch)."""
import pytest
import torch

import oracle
from minivllm_amd.layers.fused import sample_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("batch,vocab", [(7, 1000), (64, 151936), (3, 5), (1, 4099), (130, 257)])
def test_sampler_with_given_noise_matches_oracle(dtype, batch, vocab):
    g = torch.Generator().manual_seed(batch * 1000 + vocab)
    logits = (torch.randn(batch, vocab, generator=g) * 3).to(dtype)
    temps = torch.rand(batch, generator=g) * 1.5 + 0.05
    noise = torch.empty(batch, vocab).exponential_(1.0, generator=g)
    noise[0, 0] = 0.0                                              # exercises the 1e-10 clamp
    want = oracle.sampler_oracle(logits, temps, noise)
    got = sample_tokens(logits.to(DEV), temps.to(DEV), noise=noise.to(DEV)).cpu()
    assert got.dtype == torch.int64 and torch.equal(got, want)
    one = sample_tokens(logits.to(DEV), temps.to(DEV), noise=noise.to(DEV), use_workspace=False).cpu()
    assert torch.equal(one, want)                                  # one workgroup per row: same tokens


def test_sampler_generated_noise_matches_the_counter_stream():
    """Without a noise tensor the kernel must draw exactly the documented Philox stream: feeding the oracle's
    restatement of that stream to the oracle sampler gives the same tokens."""
    batch, vocab = 33, 32003
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(batch, vocab, generator=g) * 2).to(torch.bfloat16)
    temps = torch.full((batch,), 0.6)
    for seed, offset in ((0, 0), (12345, 7), (2 ** 40 + 5, 2 ** 33 + 1)):
        noise = oracle.exponential_noise_oracle(seed, offset, batch, vocab)
        want = oracle.sampler_oracle(logits, temps, noise)
        got = sample_tokens(logits.to(DEV), temps.to(DEV), seed=seed, offset=offset).cpu()
        assert torch.equal(got, want), (seed, offset, int((got != want).sum()))
    a = sample_tokens(logits.to(DEV), temps.to(DEV), seed=1, offset=0)
    b = sample_tokens(logits.to(DEV), temps.to(DEV), seed=1, offset=1)
    assert not torch.equal(a, b)


def test_sampler_distribution_strided_rows_and_low_temperature():
    vocab = 6
    row = torch.tensor([1.5, 0.0, -0.5, 2.0, 0.7, -3.0])
    wide = torch.zeros(20000, 16)
    wide[:, :vocab] = row
    logits = wide.to(DEV)[:, :vocab]                               # row stride 16, not contiguous
    temps = torch.full((20000,), 0.9, device=DEV)
    ids = sample_tokens(logits, temps, seed=5, offset=0).cpu()
    freq = torch.bincount(ids, minlength=vocab).float() / 20000
    assert float((freq - torch.softmax(row / 0.9, dim=-1)).abs().max()) < 0.015
    cold = sample_tokens(logits[:64], torch.full((64,), 1e-4, device=DEV), seed=5, offset=1).cpu()
    assert bool((cold == 3).all())                                 # temperature -> 0 is greedy
    with pytest.raises(ValueError):
        sample_tokens(logits, temps[:5])
