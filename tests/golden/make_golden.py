#!/usr/bin/env python3
"""Writes the small golden fixtures under tests/golden/ from the CPU oracle.

Run from the repository root: ``python tests/golden/make_golden.py``.
The reference repository holds no golden vectors for this path, so these
fixtures pin the oracle itself (tests/test_golden.py fails if the oracle's
results drift) and give the GPU tests fixed inputs/outputs.  16-bit tensors are
stored as their raw uint16 bit patterns; expected attention outputs are fp32.
"""
import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
from helpers import make_paged_case, make_slot_mapping, make_varlen_case  # noqa: E402


def bits(t):
    return t.view(torch.int16).numpy().view(np.uint16) if t.dtype in (torch.bfloat16, torch.float16) else t.numpy()


def main():
    # paged decode, fp32, head_dim 64 (generic kernel), block_size 16
    hq, hkv, d, bs = 4, 2, 64, 16
    q, kc, vc, tables, ctx = make_paged_case(101, 0, 0, 0, hq, hkv, d, bs, ctx_list=[1, 17, 40, 64], extra_blocks=1)
    scale = 1 / math.sqrt(d)
    out = oracle.decode_naive_oracle(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
    np.savez(os.path.join(HERE, "decode_fp32.npz"), q=q.numpy(), k_cache=kc.numpy(), v_cache=vc.numpy(),
             block_tables=tables.numpy(), context_lens=ctx.numpy(), scale=np.float32(scale), out=out.numpy(),
             shape=np.array([hq, hkv, d, bs]))

    # paged decode, bf16, head_dim 128 (MFMA kernel), GQA 4
    hq, hkv, d, bs = 8, 2, 128, 16
    q, kc, vc, tables, ctx = make_paged_case(102, 0, 0, 0, hq, hkv, d, bs, dtype=torch.bfloat16,
                                             ctx_list=[5, 33, 130], extra_blocks=1)
    scale = 1 / math.sqrt(d)
    out = oracle.decode_naive_oracle(q.float(), kc.float(), vc.float(), tables, ctx, scale, hq, hkv, d, bs)
    np.savez(os.path.join(HERE, "decode_bf16.npz"), q=bits(q), k_cache=bits(kc), v_cache=bits(vc),
             block_tables=tables.numpy(), context_lens=ctx.numpy(), scale=np.float32(scale), out=out.numpy(),
             shape=np.array([hq, hkv, d, bs]))

    # varlen causal prefill, bf16, three prompts
    hq, hkv, d = 4, 2, 128
    lengths = [7, 64, 33]
    q, k, v, cu = make_varlen_case(103, lengths, hq, hkv, d, dtype=torch.bfloat16)
    scale = 1 / math.sqrt(d)
    out = oracle.prefill_standard_oracle(q.float(), k.float(), v.float(), cu, scale, hq, hkv, d)
    np.savez(os.path.join(HERE, "prefill_bf16.npz"), q=bits(q), k=bits(k), v=bits(v), cu_seqlens=cu.numpy(),
             scale=np.float32(scale), out=out.numpy(), shape=np.array([hq, hkv, d]))

    # INT8 store: 64 tokens, 1 % outliers at 8 sigma, one all-zero vector
    hkv, d, bs = 2, 128, 16
    g = torch.Generator().manual_seed(104)
    k = torch.randn(64, hkv, d, generator=g)
    v = torch.randn(64, hkv, d, generator=g)
    k[torch.rand(k.shape, generator=g) < 0.01] *= 8.0
    v[torch.rand(v.shape, generator=g) < 0.01] *= 8.0
    k[10, 1] = 0.0
    slots, _, nb = make_slot_mapping(105, [40, 24], bs, extra_blocks=1)
    kcodes = torch.zeros(nb, bs, hkv, d, dtype=torch.int8)
    vcodes = torch.zeros_like(kcodes)
    kscale = torch.zeros(nb, bs, hkv)
    vscale = torch.zeros_like(kscale)
    oracle.store_kvcache_int8_oracle(k, v, kcodes, vcodes, kscale, vscale, slots, bs)
    np.savez(os.path.join(HERE, "store_int8.npz"), key=k.numpy(), value=v.numpy(), slot_mapping=slots.numpy(),
             k_cache=kcodes.numpy(), v_cache=vcodes.numpy(), k_scale=kscale.numpy(), v_scale=vscale.numpy(),
             shape=np.array([hkv, d, bs, nb]))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
