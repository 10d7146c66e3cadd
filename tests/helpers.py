"""Seeded synthetic inputs shared by the CPU and GPU tests."""
from __future__ import annotations

import math

import torch


def make_paged_case(seed, batch, ctx_lo, ctx_hi, num_heads, num_kv_heads, head_dim, block_size,
                    dtype=torch.float32, extra_blocks=3, ctx_list=None, log_uniform=False):
    """Random q / caches, context lengths, and disjoint shuffled block tables (CPU tensors)."""
    g = torch.Generator().manual_seed(seed)
    if ctx_list is not None:
        ctx = torch.tensor(ctx_list, dtype=torch.int64)
    elif log_uniform:
        u = torch.rand(batch, generator=g)
        ctx = torch.exp(math.log(ctx_lo) + u * (math.log(ctx_hi) - math.log(ctx_lo))).round().to(torch.int64)
    else:
        ctx = torch.randint(ctx_lo, ctx_hi + 1, (batch,), generator=g)
    batch = ctx.numel()
    need = [int(-(-int(c) // block_size)) for c in ctx.tolist()]
    num_blocks = sum(need) + extra_blocks
    perm = torch.randperm(num_blocks, generator=g)
    width = max(max(need), 1)
    tables = torch.full((batch, width), -1, dtype=torch.int32)
    at = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[at:at + n].to(torch.int32)
        at += n
    q = torch.randn(batch, num_heads, head_dim, generator=g).to(dtype)
    k_cache = torch.randn(num_blocks, block_size, num_kv_heads, head_dim, generator=g).to(dtype)
    v_cache = torch.randn(num_blocks, block_size, num_kv_heads, head_dim, generator=g).to(dtype)
    return q, k_cache, v_cache, tables, ctx


def make_varlen_case(seed, lengths, num_heads, num_kv_heads, head_dim, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    total = int(sum(lengths))
    q = torch.randn(total, num_heads, head_dim, generator=g).to(dtype)
    k = torch.randn(total, num_kv_heads, head_dim, generator=g).to(dtype)
    v = torch.randn(total, num_kv_heads, head_dim, generator=g).to(dtype)
    cu = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
    return q, k, v, cu


def make_slot_mapping(seed, lengths, block_size, extra_blocks=2):
    """Slots laid out as the engine does: each sequence owns shuffled physical blocks,
    token i of a sequence sits at block[i // bs] * bs + i % bs."""
    g = torch.Generator().manual_seed(seed)
    need = [-(-n // block_size) for n in lengths]
    num_blocks = sum(need) + extra_blocks
    perm = torch.randperm(num_blocks, generator=g).tolist()
    slots, tables, at = [], [], 0
    for n, nb in zip(lengths, need):
        blocks = perm[at:at + nb]
        at += nb
        tables.append(blocks)
        for i in range(n):
            slots.append(blocks[i // block_size] * block_size + i % block_size)
    return torch.tensor(slots, dtype=torch.int64), tables, num_blocks


def half_step(ref, dtype):
    """Half the spacing of `dtype` (bf16: 8 significant bits, fp16: 11) at each value of `ref`: what rounding a
    result to that type may cost by itself, 2^(floor(log2 |x|) - 8) or - 11; between |x| 2^-9 and |x| 2^-8 for bf16."""
    bits = 8 if dtype == torch.bfloat16 else 11
    mag = ref.to(torch.float32).abs()
    step = torch.exp2(torch.floor(torch.log2(mag.clamp_min(2.0 ** -100))) - bits)
    return torch.where(mag > 0, step, torch.zeros_like(step))


def error_stats(out, ref):
    diff = (out.to(torch.float32) - ref.to(torch.float32)).abs()
    return diff.max().item(), diff.mean().item()


def make_paged_case_on_device(seed, device, batch, ctx_lo, ctx_hi, num_heads, num_kv_heads, head_dim, block_size,
                              dtype=torch.bfloat16, log_uniform=True):
    """Large-shape variant: caches are drawn on the device (N(0,1)); tables and lengths on the host.
    Returns (q, k_cache, v_cache, tables, ctx) with q/caches on `device`, tables/ctx on the CPU."""
    g = torch.Generator().manual_seed(seed)
    if log_uniform:
        u = torch.rand(batch, generator=g)
        ctx = torch.exp(math.log(ctx_lo) + u * (math.log(ctx_hi) - math.log(ctx_lo))).round().to(torch.int64)
    else:
        ctx = torch.randint(ctx_lo, ctx_hi + 1, (batch,), generator=g)
    need = [int(-(-int(c) // block_size)) for c in ctx.tolist()]
    num_blocks = sum(need)
    perm = torch.randperm(num_blocks, generator=g)
    tables = torch.full((batch, max(need)), -1, dtype=torch.int32)
    at = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[at:at + n].to(torch.int32)
        at += n
    dg = torch.Generator(device=device).manual_seed(seed + 1)
    q = torch.randn(batch, num_heads, head_dim, generator=dg, device=device).to(dtype)
    shape = (num_blocks, block_size, num_kv_heads, head_dim)
    k_cache = torch.empty(shape, dtype=dtype, device=device)
    v_cache = torch.empty(shape, dtype=dtype, device=device)
    step = max(1, (1 << 26) // (block_size * num_kv_heads * head_dim))
    for lo in range(0, num_blocks, step):          # chunked so the fp32 staging stays small
        hi = min(num_blocks, lo + step)
        k_cache[lo:hi] = torch.randn((hi - lo,) + shape[1:], generator=dg, device=device).to(dtype)
        v_cache[lo:hi] = torch.randn((hi - lo,) + shape[1:], generator=dg, device=device).to(dtype)
    return q, k_cache, v_cache, tables, ctx


def extract_sequence(k_cache, v_cache, tables, ctx, b, block_size):
    """Compact CPU copy of one sequence's blocks with an identity table (for the CPU oracle)."""
    need = -(-int(ctx[b]) // block_size)
    ids = tables[b, :need].long().to(k_cache.device)
    kc = k_cache[ids].cpu()
    vc = v_cache[ids].cpu()
    table = torch.arange(need, dtype=torch.int32).unsqueeze(0)
    return kc, vc, table, ctx[b:b + 1]


def make_paged_prefill_case(seed, kv_lengths, cached, num_heads, num_kv_heads, head_dim, block_size,
                            dtype=torch.float32, poison=float("nan")):
    """Sequences of ``kv_lengths`` tokens whose first ``cached`` tokens count as a cached prefix.

    Returns the full packed (q, k, v, cu_k) of a plain prefill, the caches holding every key (rows of a block
    past a sequence's end are filled with ``poison``: the kernel must not let them through), the padded block
    tables, and the query rows / cu_seqlens_q of the new tokens only.
    """
    q, k, v, cu_k = make_varlen_case(seed, kv_lengths, num_heads, num_kv_heads, head_dim, dtype)
    slots, tables, num_blocks = make_slot_mapping(seed + 1, kv_lengths, block_size)
    k_cache = torch.full((num_blocks, block_size, num_kv_heads, head_dim), poison).to(dtype)
    v_cache = torch.full((num_blocks, block_size, num_kv_heads, head_dim), poison).to(dtype)
    k_cache.view(-1, num_kv_heads, head_dim)[slots] = k
    v_cache.view(-1, num_kv_heads, head_dim)[slots] = v
    width = max(len(t) for t in tables)
    block_tables = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32)
    new_rows = torch.cat([torch.arange(int(cu_k[s]) + c, int(cu_k[s + 1])) for s, c in enumerate(cached)])
    cu_q = torch.zeros(len(kv_lengths) + 1, dtype=torch.int32)
    cu_q[1:] = torch.tensor([n - c for n, c in zip(kv_lengths, cached)], dtype=torch.int32).cumsum(0)
    return dict(q=q, k=k, v=v, cu_k=cu_k, k_cache=k_cache, v_cache=v_cache, block_tables=block_tables,
                q_new=q[new_rows].contiguous(), new_rows=new_rows, cu_q=cu_q)
