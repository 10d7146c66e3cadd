"""Golden fixtures: the CPU oracle must reproduce them exactly (CPU), and the HIP path must match
them to the stated tolerances (GPU)."""
import pytest
import torch

import oracle
from golden_io import bf16, load, t

DEV = "cuda:0"


def test_oracle_reproduces_decode_fixtures():
    f = load("decode_fp32.npz")
    hq, hkv, d, bs = [int(x) for x in f["shape"]]
    out = oracle.decode_naive_oracle(t(f["q"]), t(f["k_cache"]), t(f["v_cache"]), t(f["block_tables"]),
                                     t(f["context_lens"]), float(f["scale"]), hq, hkv, d, bs)
    assert torch.allclose(out, t(f["out"]), atol=1e-6)
    out2 = oracle.decode_vectorised_oracle(t(f["q"]), t(f["k_cache"]), t(f["v_cache"]), t(f["block_tables"]),
                                           t(f["context_lens"]), float(f["scale"]), hq, hkv, d, bs)
    assert torch.allclose(out2, t(f["out"]), atol=1e-6)
    f = load("decode_bf16.npz")
    hq, hkv, d, bs = [int(x) for x in f["shape"]]
    out = oracle.decode_naive_oracle(bf16(f["q"]).float(), bf16(f["k_cache"]).float(), bf16(f["v_cache"]).float(),
                                     t(f["block_tables"]), t(f["context_lens"]), float(f["scale"]), hq, hkv, d, bs)
    assert torch.allclose(out, t(f["out"]), atol=1e-6)


def test_oracle_reproduces_prefill_and_int8_fixtures():
    f = load("prefill_bf16.npz")
    hq, hkv, d = [int(x) for x in f["shape"]]
    out = oracle.prefill_standard_oracle(bf16(f["q"]).float(), bf16(f["k"]).float(), bf16(f["v"]).float(),
                                         t(f["cu_seqlens"]), float(f["scale"]), hq, hkv, d)
    assert torch.allclose(out, t(f["out"]), atol=1e-6)
    f = load("store_int8.npz")
    hkv, d, bs, nb = [int(x) for x in f["shape"]]
    got = [torch.zeros(nb, bs, hkv, d, dtype=torch.int8), torch.zeros(nb, bs, hkv, d, dtype=torch.int8),
           torch.zeros(nb, bs, hkv), torch.zeros(nb, bs, hkv)]
    oracle.store_kvcache_int8_oracle(t(f["key"]), t(f["value"]), *got, t(f["slot_mapping"]), bs)
    for g, name in zip(got, ["k_cache", "v_cache", "k_scale", "v_scale"]):
        assert torch.equal(g, t(f[name])), name


@pytest.mark.gpu
def test_gpu_matches_decode_fixtures():
    from minivllm_amd.layers.attention import paged_attention_decode
    f = load("decode_fp32.npz")
    hq, hkv, d, bs = [int(x) for x in f["shape"]]
    out = paged_attention_decode(t(f["q"]).to(DEV), t(f["k_cache"]).to(DEV), t(f["v_cache"]).to(DEV),
                                 t(f["block_tables"]).to(DEV), t(f["context_lens"]).to(DEV), float(f["scale"]),
                                 hq, hkv, d, bs).cpu()
    assert (out - t(f["out"])).abs().max() <= 2e-4
    f = load("decode_bf16.npz")
    hq, hkv, d, bs = [int(x) for x in f["shape"]]
    out = paged_attention_decode(bf16(f["q"]).to(DEV), bf16(f["k_cache"]).to(DEV), bf16(f["v_cache"]).to(DEV),
                                 t(f["block_tables"]).to(DEV), t(f["context_lens"]).to(DEV), float(f["scale"]),
                                 hq, hkv, d, bs).cpu().float()
    err = (out - t(f["out"])).abs()
    assert err.max() <= 2e-2 and err.mean() <= 2e-3


@pytest.mark.gpu
def test_gpu_matches_prefill_and_int8_fixtures():
    from minivllm_amd.layers.attention import flash_attention_prefill, store_kvcache_int8
    f = load("prefill_bf16.npz")
    hq, hkv, d = [int(x) for x in f["shape"]]
    out = flash_attention_prefill(bf16(f["q"]).to(DEV), bf16(f["k"]).to(DEV), bf16(f["v"]).to(DEV),
                                  t(f["cu_seqlens"]).to(DEV), float(f["scale"]), hq, hkv, d).cpu().float()
    err = (out - t(f["out"])).abs()
    assert err.max() <= 2e-2 and err.mean() <= 2e-3
    f = load("store_int8.npz")
    hkv, d, bs, nb = [int(x) for x in f["shape"]]
    got = [torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV), torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=DEV),
           torch.zeros(nb, bs, hkv, device=DEV), torch.zeros(nb, bs, hkv, device=DEV)]
    store_kvcache_int8(t(f["key"]).to(DEV), t(f["value"]).to(DEV), *got, t(f["slot_mapping"]).to(DEV), bs)
    for g, name in zip(got, ["k_cache", "v_cache", "k_scale", "v_scale"]):
        assert torch.equal(g.cpu(), t(f[name])), name
