"""mvllm_paged_decode_noalloc (split-K partials in the library's static device array) against
mvllm_paged_decode (caller-owned workspace): the same kernels on the same plan, so the outputs must be
bit-identical.  Two calls in a row share the array, the second with a smaller input; every call goes
through the C ABI."""
import math

import pytest
import torch

from helpers import make_paged_case
from minivllm_amd import _C
from minivllm_amd.layers.attention import paged_attention_decode, paged_decode_plan

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NOALLOC_MAX_BYTES = 32 << 20        # MVLLM_PAGED_DECODE_NOALLOC_MAX_BYTES in include/minivllm_amd.h


def _noalloc(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs):
    out = torch.empty_like(q)
    st = _C.load().mvllm_paged_decode_noalloc(
        out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), tables.data_ptr(), tables.shape[1],
        ctx.data_ptr(), int(ctx.dtype == torch.int64), q.shape[0], hq, hkv, d, bs, kc.shape[0], float(scale),
        _C.dtype_code(q.dtype), _C.current_stream_ptr(q.device))
    return st, out


def _case(seed, batch, ctx_lo, ctx_hi, hq, hkv, d, bs, width_tokens):
    q, kc, vc, tables, ctx = make_paged_case(seed, batch, ctx_lo, ctx_hi, hq, hkv, d, bs, dtype=torch.bfloat16)
    wide = torch.full((batch, width_tokens // bs), -1, dtype=torch.int32)       # a table wider than any context
    wide[:, :tables.shape[1]] = tables
    return [t.to(DEV) for t in (q, kc, vc, wide, ctx)]


def test_noalloc_matches_workspace_entry_two_calls():
    hq, hkv, d, bs = 32, 8, 128, 16
    scale = 1 / math.sqrt(d)
    lib = _C.load()
    # first call: 12 sequences of up to 7000 tokens in an 8192-token table; second call: 5 sequences of up to 3000
    for seed, batch, hi in ((41, 12, 7000), (42, 5, 3000)):
        q, kc, vc, tables, ctx = _case(seed, batch, 40, hi, hq, hkv, d, bs, 8192)
        plan = paged_decode_plan(batch, hq, hkv, d, tables.shape[1], bs)
        assert plan[1] > 1, plan                                   # several partitions: the scratch is in use
        need = lib.mvllm_paged_decode_workspace_bytes(batch, hq, d, tables.shape[1], bs)
        assert 0 < need <= NOALLOC_MAX_BYTES
        want = paged_attention_decode(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
        st, got = _noalloc(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
        torch.cuda.synchronize()
        assert st == 0
        assert torch.equal(got, want), (seed, (got.float() - want.float()).abs().max().item())


def test_noalloc_rejects_shapes_beyond_the_static_array():
    hq, hkv, d, bs = 32, 8, 128, 16
    lib = _C.load()
    batch, blocks = 256, 2048                                      # 256 x 32 partitions x 32 heads: 136 MB of partials
    assert lib.mvllm_paged_decode_workspace_bytes(batch, hq, d, blocks, bs) > NOALLOC_MAX_BYTES
    q = torch.zeros(batch, hq, d, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(4, bs, hkv, d, dtype=torch.bfloat16, device=DEV)
    tables = torch.full((batch, blocks), -1, dtype=torch.int32, device=DEV)
    ctx = torch.zeros(batch, dtype=torch.int32, device=DEV)
    st, _ = _noalloc(q, kc, kc, tables, ctx, 1.0, hq, hkv, d, bs)
    assert st == -5                                                # MVLLM_ERR_WORKSPACE, nothing launched
    with pytest.raises(ValueError):
        _C.check(st, "paged_decode_noalloc")


def test_noalloc_allocates_nothing():
    """Device memory in use is the same before and after a call (the partials live in the library's static array, not
    in an allocation), and the call can be recorded into a graph, where an allocation would fail the capture; every
    replay equals the eager result."""
    hq, hkv, d, bs = 32, 8, 128, 16
    scale = 1 / math.sqrt(d)
    q, kc, vc, tables, ctx = _case(43, 9, 40, 6000, hq, hkv, d, bs, 8192)
    out = torch.empty_like(q)
    lib = _C.load()

    def call():
        return lib.mvllm_paged_decode_noalloc(
            out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), tables.data_ptr(), tables.shape[1],
            ctx.data_ptr(), int(ctx.dtype == torch.int64), q.shape[0], hq, hkv, d, bs, kc.shape[0], float(scale),
            _C.dtype_code(q.dtype), _C.current_stream_ptr(q.device))

    assert call() == 0                                             # first call on the device: the symbol lookup
    torch.cuda.synchronize()
    want = out.clone()
    free_before, _ = torch.cuda.mem_get_info()
    assert call() == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    assert torch.equal(out, want)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert call() == 0
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
