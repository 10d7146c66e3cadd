"""lm_head_sample (LM head + sampler in one pass over the weights) against the two steps it replaces:
``sample_tokens(F.linear(hidden, weight))`` with the same seed and offset.  The noise stream is the same (same Philox
counters), the logits are rounded to the element type in both, and only the order of the fp32 sums inside a logit
differs (library GEMM against this kernel): a logit can land on the neighbouring 16-bit value now and then, which
changes a row's winner only when its two best scores are that close.  Asserted: at least 95 % of the rows agree (all
of them did when this was written), and rows with one dominant logit agree always."""
import pytest
import torch
import torch.nn.functional as F

from minivllm_amd.layers.fused import (lm_head_sample, lm_head_sample_takes, lm_head_sample_workspace_bytes,
                                       sample_tokens)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, m, vocab, k, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(dtype).to(DEV)
    w = (torch.randn(vocab, k, generator=g) * 0.05).to(dtype).to(DEV)
    t = (0.3 + torch.rand(m, generator=g)).to(DEV)
    return x, w, t


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m", [1, 7, 16, 17, 40, 64])
@pytest.mark.parametrize("vocab,k", [(151936, 1024), (2048, 256), (4112, 512)])
def test_lm_head_sample_equals_gemm_then_sampler(dtype, m, vocab, k):
    x, w, t = _case(500 + m, m, vocab, k, dtype)
    assert lm_head_sample_takes(x, w)
    agree = total = 0
    for offset in (0, 3, 1 << 33):
        want = sample_tokens(F.linear(x, w), t, seed=11, offset=offset)
        got = lm_head_sample(x, w, t, seed=11, offset=offset)
        assert got.dtype == torch.int64 and bool(((got >= 0) & (got < vocab)).all())
        agree += int((got == want).sum())
        total += m
    assert agree >= 0.95 * total, (agree, total)
    # one logit far above the rest: the winner does not depend on the last bit of anything
    xs = x.clone()
    winners = torch.randint(0, vocab, (m,), generator=torch.Generator().manual_seed(m)).to(DEV)
    xs[:] = (w[winners].float() * 40).to(dtype)               # row b is 40 x the weight row of its winner
    assert torch.equal(lm_head_sample(xs, w, t, seed=1, offset=0), winners)


def test_row_index_picks_the_rows_and_device_offset_draws_fresh_noise():
    x, w, t = _case(77, 48, 4096, 1024, torch.bfloat16)
    rows = torch.tensor([47, 0, 13, 13, 5], device=DEV)
    t5 = t[:5].contiguous()
    want = lm_head_sample(x[rows].contiguous(), w, t5, seed=3, offset=8)
    got = lm_head_sample(x, w, t5, seed=3, offset=8, row_index=rows)
    assert torch.equal(got, want)
    # rows 2 and 3 read the same hidden row but are different rows of the batch: their noise differs
    step = torch.tensor([8], dtype=torch.int64, device=DEV)
    ws = torch.empty(lm_head_sample_workspace_bytes(5, 1024), dtype=torch.uint8, device=DEV)
    out = torch.empty(5, dtype=torch.int64, device=DEV)
    lm_head_sample(x, w, t5, seed=3, offset=0, row_index=rows, out=out, offset_dev=step, workspace=ws)
    assert torch.equal(out, want)                             # offset 0 + the counter's 8
    step += 1
    lm_head_sample(x, w, t5, seed=3, offset=0, row_index=rows, out=out, offset_dev=step, workspace=ws)
    assert torch.equal(out, lm_head_sample(x, w, t5, seed=3, offset=9, row_index=rows))
    assert not lm_head_sample_takes(x.float(), w.float())
    assert not lm_head_sample_takes(torch.zeros(65, 1024, dtype=torch.bfloat16, device=DEV), w)
    assert not lm_head_sample_takes(x, w[:4090])              # vocabulary not a multiple of 16
    with pytest.raises(ValueError):
        lm_head_sample(x, w[:4090], t, seed=0)


def test_lm_head_sample_follows_the_tempered_distribution():
    """Frequencies over many call offsets against softmax(logits / T) on a small vocabulary (one hidden row repeated
    in 64 rows of the batch: 64 independent draws per call)."""
    vocab, k, m = 64, 256, 64
    g = torch.Generator().manual_seed(5)
    row = torch.randn(1, k, generator=g)
    x = row.repeat(m, 1).to(torch.bfloat16).to(DEV)
    w = (torch.randn(vocab, k, generator=g) * 0.12).to(torch.bfloat16).to(DEV)
    t = torch.full((m,), 0.8, device=DEV)
    logits = F.linear(x[:1], w).float()
    probs = torch.softmax(logits / 0.8, dim=-1)[0].cpu()
    counts = torch.zeros(vocab)
    calls = 400
    for off in range(calls):
        ids = lm_head_sample(x, w, t, seed=21, offset=off).cpu()
        counts += torch.bincount(ids, minlength=vocab).float()
    freq = counts / (calls * m)
    # 25 600 draws: the standard error of a frequency p is sqrt(p (1 - p) / n) <= 0.0031; five of them
    assert float((freq - probs).abs().max()) <= 5 * float((probs * (1 - probs) / (calls * m)).sqrt().max()) + 1e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_lm_head_sample_against_the_cpu_oracle(dtype):
    """Against the oracle end to end: fp32 product of the 16-bit operands on the CPU rounded to the element type
    (the LM head's logits), the oracle's restatement of the Philox noise stream, and the oracle's sampler.  The fp32
    sums may differ in their last bits, so a row may differ where its two best scores nearly tie: at least 95 % of the
    rows equal (all of them when this was written)."""
    import oracle
    agree = total = 0
    for seed, m, vocab, k, offset in [(1, 5, 2048, 256, 0), (2, 33, 4096, 512, 7), (3, 64, 1024, 1024, (1 << 32) + 5)]:
        x, w, t = _case(900 + seed, m, vocab, k, dtype)
        logits = (x.float().cpu() @ w.float().cpu().T).to(dtype)
        noise = oracle.exponential_noise_oracle(40 + seed, offset, m, vocab)
        want = oracle.sampler_oracle(logits, t.cpu(), noise)
        got = lm_head_sample(x, w, t, seed=40 + seed, offset=offset).cpu()
        agree += int((got == want).sum())
        total += m
    assert agree >= 0.95 * total, (agree, total)
