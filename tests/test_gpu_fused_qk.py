"""qk_norm_rope_store on the GPU vs the CPU oracle of the unfused chain (RMSNorm -> rotary -> store).

Tolerance: the kernel rounds where the chain rounds (after the norm, after the rotation) and uses separate IEEE
multiplies/adds, so only the order of the sum of squares differs from the oracle.  A different last bit of that
sum can move a result by one unit in the last place of the element type; everything else must be identical:
 * without the norm (no sum): bit-exact;
 * with the norm: for bf16/fp16 at least 99.5 % of the elements bit-exact, the rest (and every fp32 element)
   within 1 ulp (2^-7 relative for bf16, 2^-10 for fp16; 2^-22 for fp32) of the result plus as much of the
   rotated pair's magnitude;
 * cache contents: bit-exact against the oracle's store applied to the kernel's own k_out / v (codes and
   scales included).
"""
import pytest
import torch

import oracle
from helpers import make_slot_mapping
from minivllm_amd.layers.fused import qk_norm_rope_store

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ULP = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.0 ** -22}


def _case(seed, t, hq, hkv, d, dtype, max_pos=512):
    g = torch.Generator().manual_seed(seed)
    qkv = torch.randn(t, (hq + 2 * hkv) * d, generator=g).to(dtype)       # the packed projection output
    q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    q, k, v = q.unflatten(-1, (hq, d)), k.unflatten(-1, (hkv, d)), v.unflatten(-1, (hkv, d))
    pos = torch.randint(0, max_pos, (t,), generator=g)
    gamma = (torch.rand(d, generator=g) + 0.5).float()
    table = oracle.rope_cos_sin_cache_oracle(1e6, d, max_pos)
    return qkv, (q, k, v), pos, gamma, table


def _dev_views(qkv, hq, hkv, d):
    qkv = qkv.to(DEV)
    q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    return q.unflatten(-1, (hq, d)), k.unflatten(-1, (hkv, d)), v.unflatten(-1, (hkv, d))


def _close(got, want, dtype, exact, normed=None):
    """``normed``: the oracle's norm output the rotation started from.  One ulp of it moves a rotated element by
    up to one ulp of the pair's magnitude (|x1| + |x2|), which can exceed the ulp of a result that cancelled."""
    got = got.cpu()
    if exact:
        assert torch.equal(got.view(torch.uint8), want.contiguous().view(torch.uint8))
        return
    if dtype != torch.float32:      # fp32 has no final rounding that would absorb the last bit of the sum
        same = (got == want).float().mean().item()
        assert same >= 0.995, f"only {same:.4f} of the elements are bit-exact"
    err = (got.float() - want.float()).abs()
    n1, n2 = normed.float().abs().chunk(2, dim=-1)
    pair = torch.cat([n1 + n2, n1 + n2], dim=-1)
    bound = (want.float().abs() + pair) * ULP[dtype] + 1e-30
    assert bool((err <= bound).all()), f"max excess {(err - bound).max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (4, 4, 64), (2, 1, 96), (3, 1, 256), (2, 2, 8)])
@pytest.mark.parametrize("norm", [True, False])
def test_fused_outputs_and_store(dtype, hq, hkv, d, norm):
    bs = 16
    lengths = [33, 1, 70]
    t = sum(lengths)
    slots, _, nb = make_slot_mapping(3, lengths, bs)
    slots[7] = -1
    qkv, (q, k, v), pos, gamma, table = _case(1, t, hq, hkv, d, dtype)
    gm = gamma if norm else None
    want_q, want_k = oracle.qk_norm_rope_store_oracle(q, k, v, pos, table, gm, 1e-6)
    kc = torch.full((nb, bs, hkv, d), 3.0).to(dtype).to(DEV)
    vc = torch.full((nb, bs, hkv, d), -5.0).to(dtype).to(DEV)
    dq, dk, dv = _dev_views(qkv, hq, hkv, d)
    got_q, got_k, got_v = qk_norm_rope_store(dq, dk, dv, pos.to(DEV), table.to(DEV), None if gm is None else gm.to(DEV),
                                             1e-6, slots.to(DEV), kc, vc)
    torch.cuda.synchronize()
    _close(got_q, want_q, dtype, not norm, oracle.rms_norm_oracle(q, gamma, 1e-6))
    _close(got_k, want_k, dtype, not norm, oracle.rms_norm_oracle(k, gamma, 1e-6))
    assert torch.equal(got_v.cpu(), v.contiguous())
    # the cache holds exactly what store_kvcache would write from the kernel's own outputs
    ref_k = torch.full((nb, bs, hkv, d), 3.0).to(dtype)
    ref_v = torch.full((nb, bs, hkv, d), -5.0).to(dtype)
    oracle.store_kvcache_oracle(got_k.cpu(), got_v.cpu(), ref_k, ref_v, slots, bs)
    assert torch.equal(kc.cpu().view(torch.uint8), ref_k.view(torch.uint8))
    assert torch.equal(vc.cpu().view(torch.uint8), ref_v.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (2, 1, 96)])
def test_fused_int8_cache_bit_exact(dtype, hq, hkv, d):
    bs = 16
    lengths = [40, 9]
    t = sum(lengths)
    slots, _, nb = make_slot_mapping(5, lengths, bs)
    slots[0] = -1
    qkv, (q, k, v), pos, gamma, table = _case(2, t, hq, hkv, d, dtype)
    qkv[3] = 0                                     # an all-zero token: scale 0, codes 0
    kc = torch.full((nb, bs, hkv, d), 7, dtype=torch.int8, device=DEV)
    vc = torch.full((nb, bs, hkv, d), -7, dtype=torch.int8, device=DEV)
    ks = torch.full((nb, bs, hkv), 9.0, device=DEV)
    vs = torch.full((nb, bs, hkv), -9.0, device=DEV)
    dq, dk, dv = _dev_views(qkv, hq, hkv, d)
    got_q, got_k, got_v = qk_norm_rope_store(dq, dk, dv, pos.to(DEV), table.to(DEV), gamma.to(DEV), 1e-6,
                                             slots.to(DEV), kc, vc, ks, vs)
    torch.cuda.synchronize()
    rk = torch.full((nb, bs, hkv, d), 7, dtype=torch.int8); rv = torch.full((nb, bs, hkv, d), -7, dtype=torch.int8)
    rks = torch.full((nb, bs, hkv), 9.0); rvs = torch.full((nb, bs, hkv), -9.0)
    oracle.store_kvcache_int8_oracle(got_k.cpu(), got_v.cpu(), rk, rv, rks, rvs, slots, bs)
    assert torch.equal(kc.cpu(), rk) and torch.equal(vc.cpu(), rv)
    assert torch.equal(ks.cpu(), rks) and torch.equal(vs.cpu(), rvs)


def test_fused_decode_shape_without_dense_kv_and_without_store():
    hq, hkv, d, dtype = 16, 8, 128, torch.bfloat16
    qkv, (q, k, v), pos, gamma, table = _case(4, 5, hq, hkv, d, dtype)
    dq, dk, dv = _dev_views(qkv, hq, hkv, d)
    got_q, got_k, got_v = qk_norm_rope_store(dq, dk, dv, pos.to(DEV), table.to(DEV), gamma.to(DEV), 1e-6, need_kv=False)
    torch.cuda.synchronize()
    assert got_k is None and got_v is None
    want_q, _ = oracle.qk_norm_rope_store_oracle(q, k, v, pos, table, gamma, 1e-6)
    _close(got_q, want_q, dtype, False, oracle.rms_norm_oracle(q, gamma, 1e-6))


def test_fused_positions_are_clamped_and_empty_batch():
    hq, hkv, d, dtype = 4, 2, 64, torch.float16
    qkv, (q, k, v), pos, gamma, table = _case(6, 4, hq, hkv, d, dtype, max_pos=32)
    wild = torch.tensor([-3, 31, 32, 10 ** 9])
    dq, dk, dv = _dev_views(qkv, hq, hkv, d)
    got_q, _, _ = qk_norm_rope_store(dq, dk, dv, wild.to(DEV), table.to(DEV), None)
    want_q, _ = oracle.qk_norm_rope_store_oracle(q, k, v, wild.clamp(0, 31), table, None, 0.0)
    assert torch.equal(got_q.cpu(), want_q)
    e = torch.empty(0, hq, d, dtype=dtype, device=DEV)
    ekv = torch.empty(0, hkv, d, dtype=dtype, device=DEV)
    out = qk_norm_rope_store(e, ekv, ekv, torch.empty(0, dtype=torch.long, device=DEV), table.to(DEV), None)
    assert out[0].shape == (0, hq, d)


def test_fused_rejects_bad_arguments():
    hq, hkv, d, dtype = 4, 2, 64, torch.bfloat16
    qkv, (q, k, v), pos, gamma, table = _case(7, 3, hq, hkv, d, dtype)
    dq, dk, dv = _dev_views(qkv, hq, hkv, d)
    with pytest.raises(ValueError):
        qk_norm_rope_store(dq, dk, dv, pos[:2].to(DEV), table.to(DEV), None)                 # positions size
    with pytest.raises(ValueError):
        qk_norm_rope_store(dq, dk, dv, pos.to(DEV), table.to(DEV).half(), None)              # table dtype
    with pytest.raises(ValueError):
        qk_norm_rope_store(dq.transpose(1, 2), dk, dv, pos.to(DEV), table.to(DEV), None)     # layout
    with pytest.raises(RuntimeError):
        qk_norm_rope_store(q, k, v, pos, table, None)                                         # CPU tensors
