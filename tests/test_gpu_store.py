"""store_kvcache / store_kvcache_int8 on the GPU vs the CPU oracle: bit-exact."""
import pytest
import torch

import oracle
from helpers import make_slot_mapping
from minivllm_amd.layers.attention import store_kvcache, store_kvcache_int8

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rows(seed, t, hkv, d, dtype, outliers=False):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(t, hkv, d, generator=g)
    v = torch.randn(t, hkv, d, generator=g)
    if outliers:
        k[torch.rand(k.shape, generator=g) < 0.01] *= 8.0
        v[torch.rand(v.shape, generator=g) < 0.01] *= 8.0
    return k.to(dtype), v.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hkv,d,bs", [(8, 128, 256), (2, 64, 16), (1, 5, 4), (3, 12, 8)])
def test_store_bit_exact(dtype, hkv, d, bs):
    lengths = [37, 1, 300, 16]
    slots, _, nb = make_slot_mapping(21, lengths, bs)
    t = sum(lengths)
    slots[5] = -1
    slots[t - 1] = -1
    k, v = _rows(22, t, hkv, d, dtype)
    poison_k = torch.full((nb, bs, hkv, d), 3.0).to(dtype)
    poison_v = torch.full((nb, bs, hkv, d), -5.0).to(dtype)
    want_k, want_v = poison_k.clone(), poison_v.clone()
    oracle.store_kvcache_oracle(k, v, want_k, want_v, slots, bs)
    got_k, got_v = poison_k.to(DEV), poison_v.to(DEV)
    store_kvcache(k.to(DEV), v.to(DEV), got_k, got_v, slots.to(DEV), bs)
    torch.cuda.synchronize()
    assert torch.equal(got_k.cpu().view(torch.uint8), want_k.view(torch.uint8))
    assert torch.equal(got_v.cpu().view(torch.uint8), want_v.view(torch.uint8))


def test_store_non_contiguous_inputs_and_int32_slots_and_empty():
    hkv, d, bs = 4, 32, 16
    lengths = [20, 9]
    slots, _, nb = make_slot_mapping(23, lengths, bs)
    t = sum(lengths)
    g = torch.Generator().manual_seed(24)
    qkv = torch.randn(t, 3 * hkv * d, generator=g).to(torch.bfloat16)
    k = qkv[:, hkv * d:2 * hkv * d].view(t, hkv, d)          # strided view, like a split QKV projection
    v = qkv[:, 2 * hkv * d:].view(t, hkv, d)
    want_k = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16)
    want_v = torch.zeros_like(want_k)
    oracle.store_kvcache_oracle(k, v, want_k, want_v, slots, bs)
    qkv_d = qkv.to(DEV)
    kd = qkv_d[:, hkv * d:2 * hkv * d].view(t, hkv, d)
    vd = qkv_d[:, 2 * hkv * d:].view(t, hkv, d)
    got_k = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=DEV)
    got_v = torch.zeros_like(got_k)
    store_kvcache(kd, vd, got_k, got_v, slots.to(torch.int32).to(DEV), bs)
    assert torch.equal(got_k.cpu(), want_k) and torch.equal(got_v.cpu(), want_v)
    # zero tokens: nothing happens
    store_kvcache(kd[:0], vd[:0], got_k, got_v, slots[:0].to(DEV), bs)
    assert torch.equal(got_k.cpu(), want_k)


def test_store_full_size_round_trip():
    """BASELINE.json config 2 shape: 16 prompts, L in [64, 2048], Hkv 8, D 128, bf16, block 256."""
    g = torch.Generator().manual_seed(25)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    bs, hkv, d = 256, 8, 128
    slots, tables, nb = make_slot_mapping(26, lengths, bs)
    t = sum(lengths)
    k = torch.randn(t, hkv, d, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(t, hkv, d, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    store_kvcache(k, v, kc, vc, slots.to(DEV), bs)
    sl = slots.to(DEV)
    assert torch.equal(kc.view(-1, hkv, d)[sl], k) and torch.equal(vc.view(-1, hkv, d)[sl], v)
    # nothing else was touched: number of non-zero rows == T (random rows are never all-zero)
    assert int((kc.view(nb * bs, -1) != 0).any(dim=1).sum()) == t


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hkv,d,bs", [(8, 128, 256), (2, 64, 16), (3, 96, 8), (1, 8, 4), (2, 256, 16)])
def test_store_int8_bit_exact(dtype, hkv, d, bs):
    lengths = [33, 64, 2, 150]
    slots, _, nb = make_slot_mapping(27, lengths, bs)
    t = sum(lengths)
    slots[11] = -1
    k, v = _rows(28, t, hkv, d, dtype, outliers=True)
    k[4, 0] = 0                                            # all-zero vector -> scale 0, codes 0
    v[9] = 0
    want = [torch.full((nb, bs, hkv, d), 9, dtype=torch.int8), torch.full((nb, bs, hkv, d), -9, dtype=torch.int8),
            torch.full((nb, bs, hkv), 2.5), torch.full((nb, bs, hkv), -2.5)]
    got = [w.clone().to(DEV) for w in want]
    oracle.store_kvcache_int8_oracle(k, v, *want, slots, bs)
    store_kvcache_int8(k.to(DEV), v.to(DEV), *got, slots.to(DEV), bs)
    for name, a, b in zip(["k codes", "v codes", "k scales", "v scales"], got, want):
        a = a.cpu()
        if a.dtype == torch.float32:
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name
        else:
            assert torch.equal(a, b), f"{name}: {(a != b).sum().item()} codes differ"


def test_store_int8_full_size_invariants():
    """BASELINE.json config 4 style rows (1 % outliers at 8 sigma) at 64k tokens: spec invariants on the GPU result
    and bit-exact agreement with the oracle on the whole batch."""
    bs, hkv, d, t = 256, 8, 128, 65536
    k, v = _rows(29, t, hkv, d, torch.bfloat16, outliers=True)
    nb = t // bs
    slots = torch.randperm(t, generator=torch.Generator().manual_seed(30))
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(nb, bs, hkv, device=DEV)
    vs = torch.zeros_like(ks)
    store_kvcache_int8(k.to(DEV), v.to(DEV), kc, vc, ks, vs, slots.to(DEV), bs)
    codes, scales = oracle.quantize_int8_oracle(k)
    assert torch.equal(kc.view(-1, hkv, d)[slots.to(DEV)].cpu(), codes)
    assert torch.equal(ks.view(-1, hkv)[slots.to(DEV)].cpu(), scales)
    assert int(kc.abs().amax(-1).min()) == 127 and int(vc.abs().amax(-1).min()) == 127


def test_store_int8_codes_at_rounding_boundaries():
    """Values whose quotient x / scale lies on or within a few units in the last place of k + 1/2, where a reciprocal
    multiply and the IEEE division can round to different codes, and the divisors at the ends of the range (denormal,
    tiny, huge): the codes and scales equal the oracle's (torch's fp32 division and round-half-even) bit for bit."""
    d, hkv, bs = 128, 2, 16
    g = torch.Generator().manual_seed(77)
    rows = []
    for amax in (127.0, 100.0, 3.3, 1e-3, 7e4, 1.0 / 3.0, 2e-38, 1e-41, 3e38, 6.02e23):
        scale = torch.tensor(amax, dtype=torch.float32) / 127.0
        for _ in range(6):
            kk = torch.randint(-126, 126, (d,), generator=g).float()
            x = (kk + 0.5) * scale                                  # the quotient is k + 1/2 up to rounding
            steps = torch.randint(-3, 4, (d,), generator=g)
            for _ in range(3):                                      # ... and up to 3 units in the last place around it
                x = torch.where(steps > 0, torch.nextafter(x, torch.tensor(float("inf"))), x)
                x = torch.where(steps < 0, torch.nextafter(x, torch.tensor(float("-inf"))), x)
                steps = steps - steps.sign()
            x[int(torch.randint(0, d, (1,), generator=g))] = amax   # the vector's maximum fixes the scale
            rows.append(x)
    t = len(rows) // hkv
    k = torch.stack(rows[:t * hkv]).view(t, hkv, d)
    v = -k.flip(0)
    nb = -(-t // bs)
    slots = torch.randperm(nb * bs, generator=g)[:t]
    want = [torch.zeros(nb, bs, hkv, d, dtype=torch.int8), torch.zeros(nb, bs, hkv, d, dtype=torch.int8),
            torch.zeros(nb, bs, hkv), torch.zeros(nb, bs, hkv)]
    got = [w.clone().to(DEV) for w in want]
    oracle.store_kvcache_int8_oracle(k, v, *want, slots, bs)
    store_kvcache_int8(k.to(DEV), v.to(DEV), *got, slots.to(DEV), bs)
    for name, a, b in zip(["k codes", "v codes", "k scales", "v scales"], got, want):
        a = a.cpu()
        if a.dtype == torch.float32:
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name
        else:
            assert torch.equal(a, b), f"{name}: {(a != b).sum().item()} codes differ"
    # the case is what it claims: a good part of the quotients round differently under a reciprocal multiply
    q = k / (k.abs().amax(-1, keepdim=True) / 127.0)
    near = ((q - q.round()).abs() > 0.4999).float().mean().item()
    assert near > 0.3, near
