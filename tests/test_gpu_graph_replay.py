"""Decode calls captured in a hipGraph: every replay, with contexts, queries and block tables changed in place
between replays and eager work in between, equals the eager call bit for bit.  Both kernel forms (the table width
and batch size choose), 16-bit and INT8 caches, with and without the merge launch."""
import math

import pytest
import torch

from helpers import make_paged_case
from minivllm_amd.layers.attention import (paged_attention_decode, paged_attention_decode_int8, paged_decode_plan,
                                           store_kvcache_int8)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HQ, HKV, D, BS = 32, 8, 128, 16


def _case(seed, batch, width):
    q, kc, vc, tables, ctx = make_paged_case(seed, batch, 40, 900, HQ, HKV, D, BS, dtype=torch.bfloat16)
    wide = torch.full((batch, width // BS), -1, dtype=torch.int32)
    wide[:, :tables.shape[1]] = tables
    return q.to(DEV), kc.to(DEV), vc.to(DEV), wide.to(DEV), ctx.to(DEV)


@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("batch,width,waves,merge", [(64, 4096, 4, False), (6, 8192, 4, True), (64, 32768, 1, True)])
def test_decode_graph_replays_equal_eager(int8, batch, width, waves, merge):
    q, kc, vc, tables, ctx = _case(81, batch, width)
    part, parts, w = paged_decode_plan(batch, HQ, HKV, D, width // BS, BS, torch.bfloat16, int8_cache=int8)
    assert w == waves and (parts > 1) == merge
    scale = 1 / math.sqrt(D)
    if int8:
        nb = kc.shape[0]
        ck, cv = (torch.zeros(nb, BS, HKV, D, dtype=torch.int8, device=DEV) for _ in range(2))
        sk, sv = (torch.zeros(nb, BS, HKV, device=DEV) for _ in range(2))
        store_kvcache_int8(kc.view(-1, HKV, D), vc.view(-1, HKV, D), ck, cv, sk, sv, torch.arange(nb * BS, device=DEV), BS)
        call = lambda: paged_attention_decode_int8(q, ck, cv, sk, sv, tables, ctx, scale, HQ, HKV, D, BS)
    else:
        call = lambda: paged_attention_decode(q, kc, vc, tables, ctx, scale, HQ, HKV, D, BS)
    call()                                             # the workspace is allocated outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call()
    g = torch.Generator().manual_seed(82)
    for step in range(4):
        # the engine's edits between steps: contexts grow or shrink, a sequence empties, queries change,
        # two sequences swap their blocks
        new_ctx = torch.randint(1, 901, (batch,), generator=g)
        new_ctx[step % batch] = 0
        ctx.copy_(new_ctx.to(DEV))
        q.copy_(torch.randn(q.shape, generator=g).to(torch.bfloat16).to(DEV))
        rows = tables[[0, 1]].clone()
        tables[0].copy_(rows[1])
        tables[1].copy_(rows[0])
        graph.replay()
        torch.cuda.synchronize()
        eager = call()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), step
        assert torch.count_nonzero(out[step % batch]) == 0
        _ = (kc.float().sum(), eager.float().abs().max().item())      # unrelated eager work between replays
