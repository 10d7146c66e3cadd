#!/usr/bin/env python3
"""Benchmark of the paged-attention hot path on one MI355X.

Prints ONE JSON line.  The headline (`metric`/`value`) is BASELINE.json config 3:
paged-attention decode, batch 256, context lengths log-uniform in [128, 32768],
32 query heads / 8 KV heads / head_dim 128, bf16 cache, block_size 16, reported
as algorithmic HBM GB/s.  A "step" is one decode call over the whole batch with
all inputs resident in HBM.  `extra` carries the other measured workloads
(decode at block_size 256, varlen prefill TFLOP/s and store_kvcache GB/s on
config 2, the INT8 cache path of config 4, the engine generate loop of config 5).  `cpu_baseline` times the CPU oracle's naive decode on a bounded
subset of the same batch on the host cores.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# HBM bytes one decode_mfma_kernel launch moves on the default workload (seed 0, block_size 16), from the
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in profiles/bench_hbm_traffic_pmc.txt:
# 2708744 KiB x 2.0 (copy-kernel calibration) fetched + 22855 KiB written.
DECODE_TRAFFIC_BYTES_DEFAULT = int(2708744 * 2.0 * 1024 + 22855 * 1024)
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--block-size", type=int, default=16, help="block size of the headline decode workload")
    ap.add_argument("--only", default="", help="comma list out of decode256,prefill,prefill_long,store,int8,reference_shapes,decode_small,demo_shape,head_dims,fused_qk,sampler,mfma_probe,prefill_timeline,loads_probe,engine,engine16,engine64,cpu to restrict the extras (the headline decode always runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch three 1 GiB device copies (reads 1 GiB, writes 1 GiB each) so a rocprofv3 "
                         "--pmc run can scale FETCH_SIZE / WRITE_SIZE against a kernel of known traffic")
    return ap.parse_args()


def time_steps(fn, steps, warmup, min_warm_ms=0.0):
    """W untimed calls, then K calls timed by wall clock (synchronised both sides) and by HIP events on the
    current torch stream (the stream the kernels are launched on).  Returns (wall ms/step, event ms/step).
    min_warm_ms > 0 (the `extra` legs, never the headline): warm-up calls continue until that much wall time has
    passed, because the GPU needs about 25 ms under load before its clock settles (a 0.2 ms kernel measured
    after 5 warm-up launches is 15 % slower than in steady state)."""
    import torch
    for _ in range(warmup):
        fn()
    if min_warm_ms > 0:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < min_warm_ms:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, start.elapsed_time(stop) / steps


EXTRA_WARM_MS = 50.0     # minimum warm-up of the legs under `extra` (the headline uses exactly --warmup steps)


def roofline(bound, achieved, kernel):
    """The same shape as the headline's `roofline` object, for a leg under `extra`."""
    peak, unit = (HBM_PEAK_GBS, "GB/s") if bound == "hbm" else (MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
    return {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak, "kernel": kernel}


_probe = None


def probe_lib():
    """libmvllm_probe.so with the decode entry points bound like the operator library's."""
    global _probe
    if _probe is None:
        import ctypes
        from minivllm_amd import _C
        lib = ctypes.CDLL(os.path.join(ROOT, "minivllm_amd", "libmvllm_probe.so"))
        for name in ("mvllm_paged_decode", "mvllm_paged_decode_int8", "mvllm_paged_decode_workspace_bytes"):
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = _C.SIGNATURES[name]
        _probe = lib
    return _probe


def loads_only_decode_ms(args, q, kc, vc, td, cd, scale, hq, hkv, d, bs, scales=None):
    """The same decode call on the probe library's build of the kernels, which issues every load of the real kernel
    (same grid, partitions, block-table walk, instructions) and folds the registers with xor instead of computing:
    what the access pattern alone reaches on this GPU.  Returns event ms per call."""
    import torch
    from minivllm_amd import _C
    lib = probe_lib()
    batch, mb = td.shape
    out = torch.empty_like(q)
    nbytes = lib.mvllm_paged_decode_workspace_bytes(batch, hq, d, mb, bs)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
    stream = torch.cuda.current_stream().cuda_stream
    common = (td.data_ptr(), mb, cd.data_ptr(), int(cd.dtype == torch.int64), batch, hq, hkv, d, bs, kc.shape[0],
              float(scale), _C.dtype_code(q.dtype), ws.data_ptr(), nbytes, stream)

    def call():
        if scales is None:
            st = lib.mvllm_paged_decode(out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), *common)
        else:
            st = lib.mvllm_paged_decode_int8(out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                             scales[0].data_ptr(), scales[1].data_ptr(), *common)
        assert st == 0, st
    return time_steps(call, args.steps, args.warmup, EXTRA_WARM_MS)[1]


def decode_bytes(ctx, block_size, num_heads, num_kv_heads, head_dim, kv_elem, q_elem, ctx_elem, int8_scales=False):
    """Algorithmic HBM bytes of one decode call: every live K/V element once, q read + out written once,
    one table entry per live block, one context length per sequence.  Split-K scratch is not counted."""
    tokens = int(ctx.sum())
    blocks = int(((ctx + block_size - 1) // block_size).sum())
    b = ctx.numel()
    total = tokens * num_kv_heads * head_dim * 2 * kv_elem
    if int8_scales:
        total += tokens * num_kv_heads * 2 * 4
    total += 2 * b * num_heads * head_dim * q_elem + 4 * blocks + ctx_elem * b
    return total


def bench_decode(args, block_size, want_cpu, want_probe=False):
    import torch
    from helpers import extract_sequence, make_paged_case_on_device
    from minivllm_amd.layers.attention import paged_attention_decode

    dev = "cuda:0"
    hq, hkv, d, batch = 32, 8, 128, 256
    q, kc, vc, tables, ctx = make_paged_case_on_device(args.seed, dev, batch, 128, 32768, hq, hkv, d, block_size)
    scale = 1.0 / math.sqrt(d)
    td, cd = tables.to(dev), ctx.to(dev)

    def step():
        return paged_attention_decode(q, kc, vc, td, cd, scale, hq, hkv, d, block_size)

    wall_ms, event_ms = time_steps(step, args.steps, args.warmup)
    nbytes = decode_bytes(ctx, block_size, hq, hkv, d, 2, 2, 8)
    res = {
        "workload": f"decode B256 ctx~logU[128,32768] Hq32 Hkv8 D128 bf16 block_size {block_size}",
        "tokens": int(ctx.sum()), "algorithmic_bytes": nbytes,
        "ms_per_step": wall_ms, "event_ms_per_step": event_ms,
        "gbs": nbytes / (wall_ms * 1e-3) / 1e9, "gbs_event": nbytes / (event_ms * 1e-3) / 1e9,
    }
    if want_probe:
        ms = loads_only_decode_ms(args, q, kc, vc, td, cd, scale, hq, hkv, d, block_size)
        res["loads_only"] = {"event_ms_per_step": ms, "gbs": nbytes / (ms * 1e-3) / 1e9,
                             "what": "the kernels' loads without the arithmetic (libmvllm_probe.so): the ceiling of this "
                                     "access pattern; the real kernel reaches gbs_event / this"}
    cpu = None
    if want_cpu:
        import oracle
        # bounded sample: the first sequences of the same batch up to ~24k context tokens in total
        picked, tok = [], 0
        for b in range(batch):
            if picked and tok + int(ctx[b]) > 24576:
                break
            picked.append(b)
            tok += int(ctx[b])
        parts = [extract_sequence(kc, vc, tables, ctx, b, block_size) for b in picked]
        # one compact CPU cache with per-sequence tables (block ids shifted)
        ks, vs, rows, at = [], [], [], 0
        width = max(p[2].shape[1] for p in parts)
        for k1, v1, t1, _ in parts:
            ks.append(k1.float())
            vs.append(v1.float())
            row = torch.full((width,), -1, dtype=torch.int32)
            row[:t1.shape[1]] = t1[0] + at
            rows.append(row)
            at += k1.shape[0]
        kcpu, vcpu, tcpu = torch.cat(ks), torch.cat(vs), torch.stack(rows)
        qcpu, ccpu = q[picked].float().cpu(), ctx[picked]
        oracle.decode_naive_oracle(qcpu[:1], kcpu, vcpu, tcpu[:1], ccpu[:1], scale, hq, hkv, d, block_size)
        reps, t0 = 0, time.perf_counter()
        while True:
            ref = oracle.decode_naive_oracle(qcpu, kcpu, vcpu, tcpu, ccpu, scale, hq, hkv, d, block_size)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 60:
                break
        cpu_s = (time.perf_counter() - t0) / reps
        sub_bytes = decode_bytes(ccpu, block_size, hq, hkv, d, 2, 2, 8)
        got = step()[picked].float().cpu()
        # the reference's second PyTorch path (decode_torch_optimized, benchmark_decoding.py:136-189) on the same sample
        oracle.decode_vectorised_oracle(qcpu[:1], kcpu, vcpu, tcpu[:1], ccpu[:1], scale, hq, hkv, d, block_size)
        vreps, t1 = 0, time.perf_counter()
        while True:
            ref2 = oracle.decode_vectorised_oracle(qcpu, kcpu, vcpu, tcpu, ccpu, scale, hq, hkv, d, block_size)
            vreps += 1
            if time.perf_counter() - t1 > 5.0 or vreps >= 60:
                break
        vec_s = (time.perf_counter() - t1) / vreps
        cpu = {
            "value": sub_bytes / cpu_s / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle naive decode (fp32, torch-CPU) on the first {len(picked)} sequences of the same "
                      f"batch ({tok} context tokens), {reps} reps, {cpu_s * 1e3:.1f} ms each; bf16-equivalent "
                      f"algorithmic bytes",
            "host_cpu_count": os.cpu_count(),
            "gpu_vs_oracle_max_abs": (got - ref).abs().max().item(),
            "vectorised_oracle": {"value": sub_bytes / vec_s / 1e9, "unit": "GB/s", "reps": vreps,
                                  "ms_each": vec_s * 1e3, "gpu_vs_oracle_max_abs": (got - ref2).abs().max().item()},
        }
    del kc, vc
    torch.cuda.empty_cache()
    return res, cpu


def cpu_prefill_baseline(q, k, v, cu, lengths, scale, hq, hkv, d, flops, gpu_fn):
    """The oracle's O(N^2) prefill (benchmark_prefilling.py:9-52 restated) on the whole config-2 batch on the host
    cores, fp32, timed beside the GPU; also the value check of the GPU result at full size."""
    import torch
    import oracle
    qc, kc, vc, cuc = q.float().cpu(), k.float().cpu(), v.float().cpu(), cu.cpu()
    reps, t0 = 0, time.perf_counter()
    while True:
        ref = oracle.prefill_standard_oracle(qc, kc, vc, cuc, scale, hq, hkv, d)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 5:
            break
    cpu_s = (time.perf_counter() - t0) / reps
    got = gpu_fn(q, k, v, cu, scale, hq, hkv, d).float().cpu()
    err = (got - ref).abs()
    return {"value": flops / cpu_s / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle O(N^2) prefill (fp32, torch-CPU) on the whole batch of {len(lengths)} prompts, "
                      f"{reps} reps, {cpu_s:.2f} s each; causal flops only",
            "gpu_vs_oracle_max_abs": err.max().item(), "gpu_vs_oracle_mean_abs": err.mean().item()}


def bench_prefill_store(args, which, want_cpu=False):
    """BASELINE.json config 2: 16 prompts L~U[64,2048], Hq32/Hkv8/D128 bf16; store into a block-256 paged cache."""
    import torch
    from helpers import make_slot_mapping
    from minivllm_amd.layers.attention import flash_attention_prefill, store_kvcache

    dev = "cuda:0"
    hq, hkv, d, bs = 32, 8, 128, 256
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    total = sum(lengths)
    dg = torch.Generator(device=dev).manual_seed(args.seed + 1)
    q = torch.randn(total, hq, d, generator=dg, device=dev).to(torch.bfloat16)
    k = torch.randn(total, hkv, d, generator=dg, device=dev).to(torch.bfloat16)
    v = torch.randn(total, hkv, d, generator=dg, device=dev).to(torch.bfloat16)
    cu = torch.zeros(17, dtype=torch.int32)
    cu[1:] = torch.tensor(lengths).cumsum(0)
    cu = cu.to(dev)
    out = {}
    if "prefill" in which:
        scale = 1.0 / math.sqrt(d)
        wall_ms, event_ms = time_steps(lambda: flash_attention_prefill(q, k, v, cu, scale, hq, hkv, d),
                                       args.steps, args.warmup, EXTRA_WARM_MS)
        flops = 4 * hq * d * sum(n * (n + 1) // 2 for n in lengths)
        out["prefill"] = {
            "workload": "varlen causal prefill, 16 prompts L~U[64,2048], Hq32 Hkv8 D128 bf16",
            "tokens": total, "algorithmic_flops": flops, "ms_per_step": wall_ms, "event_ms_per_step": event_ms,
            "steps": args.steps, "warmup": f"{args.warmup} launches, then at least {EXTRA_WARM_MS:.0f} ms of launches",
            "tflops": flops / (event_ms * 1e-3) / 1e12,
            "frac_of_bf16_mfma_peak": flops / (event_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "roofline": roofline("mfma", flops / (event_ms * 1e-3) / 1e12, "prefill_pp_kernel (one launch = the whole ragged batch)"),
        }
        if want_cpu:
            out["prefill"]["cpu_baseline"] = cpu_prefill_baseline(q, k, v, cu, lengths, scale, hq, hkv, d, flops,
                                                                  flash_attention_prefill)
    if "prefill" in which:
        # the same prompts on 16 query / 8 kv heads, the attention shape of the reference's model (Qwen3-0.6B): the
        # two-group kernel's items of two heads and 128 rows
        q16 = q[:, :16].contiguous()
        scale = 1.0 / math.sqrt(d)
        _, event_ms_16 = time_steps(lambda: flash_attention_prefill(q16, k, v, cu, scale, 16, hkv, d),
                                    args.steps, args.warmup, EXTRA_WARM_MS)
        flops_16 = 4 * 16 * d * sum(n * (n + 1) // 2 for n in lengths)
        out["prefill_hq16"] = {
            "workload": "the same prompts on Hq16 Hkv8 D128 bf16 (two query heads per kv head)",
            "algorithmic_flops": flops_16, "event_ms_per_step": event_ms_16, "tflops": flops_16 / (event_ms_16 * 1e-3) / 1e12,
            "roofline": roofline("mfma", flops_16 / (event_ms_16 * 1e-3) / 1e12, "prefill_pp_kernel, items of two heads"),
        }
        del q16
    if "prefill_long" in which:
        # the same kernel away from config 2's short prompts: 4 prompts of 8192 tokens (the start and end of a
        # workgroup's life are a small share of its 128 key tiles)
        long_lengths = [8192] * 4
        scale = 1.0 / math.sqrt(d)
        ql, kl, vl = (torch.randn(sum(long_lengths), h, d, generator=dg, device=dev).to(torch.bfloat16) for h in (hq, hkv, hkv))
        cul = torch.tensor([0] + long_lengths, dtype=torch.int32).cumsum(0).to(torch.int32).to(dev)
        _, event_ms_l = time_steps(lambda: flash_attention_prefill(ql, kl, vl, cul, scale, hq, hkv, d),
                                   max(3, args.steps // 4), 2, EXTRA_WARM_MS)
        flops_l = 4 * hq * d * sum(n * (n + 1) // 2 for n in long_lengths)
        out["prefill_long_prompts"] = {
            "workload": "varlen causal prefill, 4 prompts of 8192 tokens, Hq32 Hkv8 D128 bf16",
            "tokens": sum(long_lengths), "algorithmic_flops": flops_l, "event_ms_per_step": event_ms_l,
            "tflops": flops_l / (event_ms_l * 1e-3) / 1e12,
            "roofline": roofline("mfma", flops_l / (event_ms_l * 1e-3) / 1e12, "prefill_pp_kernel"),
        }
        del ql, kl, vl
        # few new tokens behind a long cached prefix (a follow-up turn): 128 tokens behind 32768 in a block-256 cache.
        # Given the host's bound on the key count the operator cuts the keys into ranges (mvllm_prefill_paged_split);
        # without it the call runs in one step, on 16 of the chip's 256 compute units.
        from minivllm_amd.layers.attention import flash_attention_prefill_paged
        new_s, prefix_s = 128, 32768
        kv_s = new_s + prefix_s
        nb_s = (kv_s + bs - 1) // bs
        kcs = torch.randn(nb_s, bs, hkv, d, generator=dg, device=dev).to(torch.bfloat16)
        vcs = torch.randn(nb_s, bs, hkv, d, generator=dg, device=dev).to(torch.bfloat16)
        qs = torch.randn(new_s, hq, d, generator=dg, device=dev).to(torch.bfloat16)
        bts = torch.randperm(nb_s, generator=torch.Generator().manual_seed(args.seed + 5)).to(torch.int32).view(1, nb_s).to(dev)
        cu_qs = torch.tensor([0, new_s], dtype=torch.int32, device=dev)
        cu_ks = torch.tensor([0, kv_s], dtype=torch.int32, device=dev)
        _, ms_split = time_steps(lambda: flash_attention_prefill_paged(qs, kcs, vcs, bts, cu_qs, cu_ks, scale, hq, hkv, d, bs,
                                                                       max_seqlen_k=kv_s),
                                 args.steps, args.warmup, EXTRA_WARM_MS)
        _, ms_one = time_steps(lambda: flash_attention_prefill_paged(qs, kcs, vcs, bts, cu_qs, cu_ks, scale, hq, hkv, d, bs),
                               max(3, args.steps // 4), 2, EXTRA_WARM_MS)
        flops_s = 4 * hq * d * (new_s * prefix_s + new_s * (new_s + 1) // 2)
        out["prefill_short_suffix"] = {
            "workload": "paged prefill of 128 new tokens behind a 32768-token cached prefix, one sequence, block_size 256, Hq32 Hkv8 D128 bf16",
            "algorithmic_flops": flops_s, "event_ms_per_step": ms_split, "tflops": flops_s / (ms_split * 1e-3) / 1e12,
            "one_step_event_ms_per_step": ms_one, "one_step_tflops": flops_s / (ms_one * 1e-3) / 1e12,
            "roofline": roofline("mfma", flops_s / (ms_split * 1e-3) / 1e12,
                                 "split_plan_kernel + prefill_mfma_kernel over key ranges + split_merge_kernel (the workspace comes from torch's allocator inside the timed call)"),
        }
        del kcs, vcs, qs
    if "prefill" in which:
        # the same prompts with the first half (whole 16-token blocks) already cached: only the second half is
        # computed, every key comes from a block-16 paged cache
        from minivllm_amd.layers.attention import flash_attention_prefill_paged
        pbs = 16
        cached = [(n // 2) // pbs * pbs for n in lengths]
        slots16, tables16, nb16 = make_slot_mapping(args.seed + 3, lengths, pbs)
        kc16 = torch.zeros(nb16, pbs, hkv, d, dtype=torch.bfloat16, device=dev)
        vc16 = torch.zeros_like(kc16)
        store_kvcache(k, v, kc16, vc16, slots16.to(dev), pbs)
        width = max(len(t) for t in tables16)
        bt = torch.tensor([t + [-1] * (width - len(t)) for t in tables16], dtype=torch.int32, device=dev)
        rows = torch.cat([torch.arange(int(cu[i]) + c, int(cu[i + 1])) for i, c in enumerate(cached)]).to(dev)
        q_new = q[rows].contiguous()
        cu_q = torch.zeros(17, dtype=torch.int32)
        cu_q[1:] = torch.tensor([n - c for n, c in zip(lengths, cached)]).cumsum(0)
        cu_q = cu_q.to(dev)
        scale = 1.0 / math.sqrt(d)
        _, event_ms = time_steps(lambda: flash_attention_prefill_paged(q_new, kc16, vc16, bt, cu_q, cu, scale, hq, hkv,
                                                                       d, pbs),
                                 args.steps, args.warmup, EXTRA_WARM_MS)
        flops = 4 * hq * d * sum((n - c) * c + (n - c) * (n - c + 1) // 2 for n, c in zip(lengths, cached))
        out["prefill_cached_prefix"] = {
            "workload": "same prompts, first half of each (whole blocks) cached: paged prefill of the rest, block_size 16",
            "new_tokens": int(cu_q[-1]), "algorithmic_flops": flops, "event_ms_per_step": event_ms,
            "tflops": flops / (event_ms * 1e-3) / 1e12,
            "frac_of_bf16_mfma_peak": flops / (event_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
            "roofline": roofline("mfma", flops / (event_ms * 1e-3) / 1e12, "prefill_pp_kernel, paged form"),
        }
        # ... and over an INT8 cache holding the same keys (codes + scales written by the INT8 store)
        from minivllm_amd.layers.attention import flash_attention_prefill_paged_int8, store_kvcache_int8
        ck8 = torch.zeros(nb16, pbs, hkv, d, dtype=torch.int8, device=dev)
        cv8 = torch.zeros_like(ck8)
        sk8 = torch.zeros(nb16, pbs, hkv, dtype=torch.float32, device=dev)
        sv8 = torch.zeros_like(sk8)
        store_kvcache_int8(k, v, ck8, cv8, sk8, sv8, slots16.to(dev), pbs)
        # in two steps (the keys and values dequantised once into a temporary 16-bit cache, then the two-group
        # kernel), which is what the operator does when the caller passes the host's max_seqlen_k; and in one step
        _, event_ms8 = time_steps(lambda: flash_attention_prefill_paged_int8(q_new, ck8, cv8, sk8, sv8, bt, cu_q, cu,
                                                                             scale, hq, hkv, d, pbs, max(lengths)),
                                  args.steps, args.warmup, EXTRA_WARM_MS)
        _, event_ms8_one = time_steps(lambda: flash_attention_prefill_paged_int8(q_new, ck8, cv8, sk8, sv8, bt, cu_q, cu,
                                                                                 scale, hq, hkv, d, pbs),
                                      args.steps, args.warmup, EXTRA_WARM_MS)
        out["prefill_cached_prefix_int8"] = {
            "workload": "the same paged prefill over an INT8 cache (codes + fp32 scales per token and kv head), block_size 16",
            "new_tokens": int(cu_q[-1]), "algorithmic_flops": flops, "event_ms_per_step": event_ms8,
            "tflops": flops / (event_ms8 * 1e-3) / 1e12,
            "one_step_event_ms_per_step": event_ms8_one, "one_step_tflops": flops / (event_ms8_one * 1e-3) / 1e12,
            "roofline": roofline("mfma", flops / (event_ms8 * 1e-3) / 1e12,
                                 "stage_blocks_kernel + prefill_pp_kernel (mvllm_prefill_paged_int8_staged; the workspace comes from torch's allocator inside the timed call)"),
        }
    if "store" in which:
        slots, _, nb = make_slot_mapping(args.seed + 2, lengths, bs)
        kc = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=dev)
        vc = torch.zeros_like(kc)
        sl = slots.to(dev)
        wall_ms, event_ms = time_steps(lambda: store_kvcache(k, v, kc, vc, sl, bs), args.steps, args.warmup, EXTRA_WARM_MS)
        nbytes = 2 * total * hkv * d * (2 + 2) + 8 * total
        out["store"] = {
            "workload": "store_kvcache of the same batch into a block-256 bf16 cache, shuffled blocks",
            "tokens": total, "algorithmic_bytes": nbytes, "ms_per_step": wall_ms, "event_ms_per_step": event_ms,
            "gbs": nbytes / (event_ms * 1e-3) / 1e9,
            "roofline": roofline("hbm", nbytes / (event_ms * 1e-3) / 1e9, "store_rows_kernel"),
        }
    return out


def bench_int8(args, want_cpu=True, want_probe=False):
    """BASELINE.json config 4: B 128, ctx U[256,16384], Hq32/Hkv8/D128; K/V ~ N(0,1) with 1 % outliers at 8 sigma are
    quantised by store_kvcache_int8 into a block-16 int8 cache, then decoded with in-kernel dequantisation."""
    import torch
    from minivllm_amd.layers.attention import paged_attention_decode_int8, store_kvcache_int8

    dev = "cuda:0"
    hq, hkv, d, batch, bs = 32, 8, 128, 128, 16
    g = torch.Generator().manual_seed(args.seed)
    ctx = torch.randint(256, 16385, (batch,), generator=g)
    need = ((ctx + bs - 1) // bs).tolist()
    nb = sum(need)
    perm = torch.randperm(nb, generator=g)
    tables = torch.full((batch, max(need)), -1, dtype=torch.int32)
    at = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[at:at + n].to(torch.int32)
        at += n
    dg = torch.Generator(device=dev).manual_seed(args.seed + 1)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=dev)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(nb, bs, hkv, dtype=torch.float32, device=dev)
    vs = torch.zeros_like(ks)
    total = nb * bs
    store_ms, chunk = [], 1 << 16
    for lo in range(0, total, chunk):                       # fill the whole cache through the INT8 store kernel
        n = min(chunk, total - lo)
        k = torch.randn(n, hkv, d, generator=dg, device=dev)
        v = torch.randn(n, hkv, d, generator=dg, device=dev)
        k = torch.where(torch.rand(k.shape, generator=dg, device=dev) < 0.01, k * 8, k).to(torch.bfloat16)
        v = torch.where(torch.rand(v.shape, generator=dg, device=dev) < 0.01, v * 8, v).to(torch.bfloat16)
        slots = torch.arange(lo, lo + n, device=dev)
        if lo == 0:
            _, ms = time_steps(lambda: store_kvcache_int8(k, v, kc, vc, ks, vs, slots, bs), args.steps, args.warmup,
                               EXTRA_WARM_MS)
            store_ms.append(ms)
            store_bytes = 2 * n * hkv * d * (2 + 1) + 8 * n + 2 * n * hkv * 4
        store_kvcache_int8(k, v, kc, vc, ks, vs, slots, bs)
    q = torch.randn(batch, hq, d, generator=dg, device=dev).to(torch.bfloat16)
    td, cd = tables.to(dev), ctx.to(dev)
    scale = 1.0 / math.sqrt(d)
    wall_ms, event_ms = time_steps(
        lambda: paged_attention_decode_int8(q, kc, vc, ks, vs, td, cd, scale, hq, hkv, d, bs),
        args.steps, args.warmup, EXTRA_WARM_MS)
    nbytes = decode_bytes(ctx, bs, hq, hkv, d, 1, 2, 8, int8_scales=True)
    check = {}
    if want_probe:
        ms = loads_only_decode_ms(args, q, kc, vc, td, cd, scale, hq, hkv, d, bs, scales=(ks, vs))
        check["loads_only"] = {"event_ms_per_step": ms, "gbs": nbytes / (ms * 1e-3) / 1e9,
                               "what": "the INT8 kernels' loads without the arithmetic (libmvllm_probe.so)"}
    if want_cpu:
        # value check at full size on the launch plan of the full batch: the longest, the shortest and six more
        # sequences against the INT8 oracle (dequantise in fp32, naive decode)
        import oracle
        got = paged_attention_decode_int8(q, kc, vc, ks, vs, td, cd, scale, hq, hkv, d, bs).float().cpu()
        order = torch.argsort(ctx)
        worst = 0.0
        for b in sorted({int(order[0]), int(order[-1]), 0, 17, 42, 64, 99, 127}):
            ids = tables[b, :need[b]].long().to(dev)
            want = oracle.decode_int8_oracle(q[b:b + 1].float().cpu(), kc[ids].cpu(), vc[ids].cpu(), ks[ids].cpu(),
                                             vs[ids].cpu(), torch.arange(need[b], dtype=torch.int32).unsqueeze(0),
                                             ctx[b:b + 1], scale, hq, hkv, d, bs)
            worst = max(worst, (got[b:b + 1] - want).abs().max().item())
        check.update({"gpu_vs_oracle_max_abs": worst, "oracle_sequences": 8})
    return {
        **check,
        "roofline": roofline("hbm", nbytes / (event_ms * 1e-3) / 1e9, "decode_mfma_int8_kernel + decode_reduce_vec_kernel"),
        "store_roofline": roofline("hbm", store_bytes / (store_ms[0] * 1e-3) / 1e9, "store_int8_kernel"),
        "workload": "INT8 KV cache: decode B128 ctx~U[256,16384] Hq32 Hkv8 D128 block_size 16, bf16 q",
        "tokens": int(ctx.sum()), "algorithmic_bytes": nbytes, "ms_per_step": wall_ms,
        "event_ms_per_step": event_ms, "gbs": nbytes / (event_ms * 1e-3) / 1e9,
        "store_int8_gbs": store_bytes / (store_ms[0] * 1e-3) / 1e9, "store_int8_tokens": chunk,
    }


def bench_fused_qk(args):
    """The caller's chain in front of the attention kernels on the prefill batch of config 2 (same lengths):
    q/k RMSNorm + rotary embedding + store into a block-256 bf16 cache, as one HIP launch reading the packed QKV
    projection output, against the same chain as separate modules (torch ops + store_kvcache)."""
    import torch
    from helpers import make_slot_mapping
    from minivllm_amd.layers.attention import store_kvcache
    from minivllm_amd.layers.basic import RMSNorm, RotaryEmbedding
    from minivllm_amd.layers.fused import qk_norm_rope_store

    dev = "cuda:0"
    hq, hkv, d, bs = 32, 8, 128, 256
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    total = sum(lengths)
    dg = torch.Generator(device=dev).manual_seed(args.seed + 1)
    qkv = torch.randn(total, (hq + 2 * hkv) * d, generator=dg, device=dev).to(torch.bfloat16)
    q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    q, k, v = q.unflatten(-1, (hq, d)), k.unflatten(-1, (hkv, d)), v.unflatten(-1, (hkv, d))
    pos = torch.cat([torch.arange(n) for n in lengths]).to(dev)
    rotary = RotaryEmbedding(1_000_000, d, 4096).to(dev)
    norm = RMSNorm(d, 1e-6).to(dev)
    gamma = norm.weight.detach().float().contiguous()
    slots, _, nb = make_slot_mapping(args.seed + 2, lengths, bs)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    sl = slots.to(dev)

    def unfused():
        qq, kk = norm(q.reshape(-1, hq, d)), norm(k.reshape(-1, hkv, d))
        qq, kk = rotary(pos, qq, kk)
        store_kvcache(kk, v.reshape(-1, hkv, d), kc, vc, sl, bs)
        return qq, kk

    fused = lambda: qk_norm_rope_store(q, k, v, pos, rotary.cos_sin_cache, gamma, 1e-6, sl, kc, vc)
    with torch.inference_mode():
        _, fused_ms = time_steps(fused, args.steps, args.warmup, EXTRA_WARM_MS)
        _, unfused_ms = time_steps(unfused, args.steps, args.warmup, EXTRA_WARM_MS)
    # read q, k, v once; write q_out, k_out, v_out and the two cache rows; per token: position, slot, table row
    nbytes = total * ((hq + 2 * hkv) * d * 2 * 2 + 2 * hkv * d * 2 + 8 + 8 + d * 4)
    return {
        "workload": "q/k RMSNorm + rotary + store_kvcache on the config-2 prefill batch, Hq32 Hkv8 D128 bf16, block 256",
        "tokens": total, "algorithmic_bytes": nbytes, "event_ms_per_step": fused_ms,
        "gbs": nbytes / (fused_ms * 1e-3) / 1e9, "unfused_modules_event_ms": unfused_ms,
        "roofline": roofline("hbm", nbytes / (fused_ms * 1e-3) / 1e9, "qk_norm_rope_store_kernel"),
    }


def bench_sampler(args):
    """One sampling step of config 5's decode batch: 64 rows of bf16 logits over the 151 936-token vocabulary,
    as one HIP launch against the module chain (fp32 softmax, exponential_, divide, argmax)."""
    import torch
    from minivllm_amd.layers.basic import Sampler
    from minivllm_amd.layers.fused import sample_tokens

    dev = "cuda:0"
    batch, vocab = 64, 151936
    dg = torch.Generator(device=dev).manual_seed(args.seed)
    logits = (torch.randn(batch, vocab, generator=dg, device=dev) * 2).to(torch.bfloat16)
    temps = torch.full((batch,), 0.6, device=dev)
    sampler = Sampler()
    _, fused_ms = time_steps(lambda: sample_tokens(logits, temps, 0, 0), args.steps, args.warmup, EXTRA_WARM_MS)
    _, modules_ms = time_steps(lambda: sampler(logits, temps, dg), args.steps, args.warmup, EXTRA_WARM_MS)
    nbytes = batch * vocab * 2 + batch * 12
    out = {"workload": "sampler: 64 x 151936 bf16 logits, T 0.6", "algorithmic_bytes": nbytes,
           "event_ms_per_step": fused_ms, "gbs": nbytes / (fused_ms * 1e-3) / 1e9, "unfused_modules_event_ms": modules_ms}
    # the LM head in front of it, config 5's: (rows, 1024) x (151936, 1024)^T, as the library GEMM + the sampler
    # launch and as one pass over the weights that never writes the logits
    import torch.nn.functional as F
    from minivllm_amd.layers.fused import lm_head_sample, lm_head_sample_workspace_bytes
    hidden_size = 1024
    w = (torch.randn(vocab, hidden_size, generator=dg, device=dev) * 0.02).to(torch.bfloat16)
    legs = {}
    for rows in (16, 64):
        x = torch.randn(rows, hidden_size, generator=dg, device=dev).to(torch.bfloat16)
        t = temps[:rows].contiguous()
        ws = torch.empty(lm_head_sample_workspace_bytes(rows, hidden_size), dtype=torch.uint8, device=dev)
        ids = torch.empty(rows, dtype=torch.int64, device=dev)
        _, one_ms = time_steps(lambda: lm_head_sample(x, w, t, 0, 0, out=ids, workspace=ws), args.steps, args.warmup,
                               EXTRA_WARM_MS)
        _, two_ms = time_steps(lambda: sample_tokens(F.linear(x, w), t, 0, 0), args.steps, args.warmup, EXTRA_WARM_MS)
        wbytes = vocab * hidden_size * 2 + rows * hidden_size * 2 + rows * 12
        same = float((lm_head_sample(x, w, t, 0, 0) == sample_tokens(F.linear(x, w), t, 0, 0)).float().mean())
        legs[f"rows{rows}"] = {"event_ms_per_step": one_ms, "gemm_then_sampler_event_ms": two_ms,
                               "ids_equal_to_gemm_then_sampler": same,
                               "roofline": roofline("hbm", wbytes / (one_ms * 1e-3) / 1e9,
                                                    "lm_head_sample_kernel + sample_combine_kernel")}
    out["lm_head_sample"] = dict(workload="LM head + sampler in one pass: rows x 1024 hidden, 151936 x 1024 bf16 weights",
                                 algorithmic_bytes=vocab * hidden_size * 2, **legs)
    return out


def bench_decode_small(args):
    """A serving-size decode call: 64 sequences of 96-352 tokens whose block table is 4096 tokens wide (the model
    length, not the contexts), 16-bit and INT8 caches, timed as 20 calls inside one hipGraph (a call is latency,
    not bandwidth, so back-to-back launches from the host would measure the host)."""
    import torch
    from helpers import make_paged_case_on_device
    from minivllm_amd.layers.attention import (paged_attention_decode, paged_attention_decode_int8, paged_decode_plan,
                                               store_kvcache_int8)

    dev = "cuda:0"
    hq, hkv, d, bs, batch, width = 32, 8, 128, 16, 64, 4096
    q, kc, vc, tables, ctx = make_paged_case_on_device(args.seed, dev, batch, 96, 352, hq, hkv, d, bs, log_uniform=False)
    wide = torch.full((batch, width // bs), -1, dtype=torch.int32)
    wide[:, :tables.shape[1]] = tables
    td, cd = wide.to(dev), ctx.to(dev)
    nb = kc.shape[0]
    ck, cv = (torch.zeros(nb, bs, hkv, d, dtype=torch.int8, device=dev) for _ in range(2))
    sk, sv = (torch.zeros(nb, bs, hkv, device=dev) for _ in range(2))
    store_kvcache_int8(kc.view(-1, hkv, d), vc.view(-1, hkv, d), ck, cv, sk, sv, torch.arange(nb * bs, device=dev), bs)
    scale = 1 / math.sqrt(d)
    calls = 20

    def graph_us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(calls):
                fn()
        _, ms = time_steps(g.replay, args.steps, 2, EXTRA_WARM_MS)
        return ms * 1e3 / calls

    us16 = graph_us(lambda: paged_attention_decode(q, kc, vc, td, cd, scale, hq, hkv, d, bs))
    us8 = graph_us(lambda: paged_attention_decode_int8(q, ck, cv, sk, sv, td, cd, scale, hq, hkv, d, bs))
    tokens = int(ctx.sum())
    return {"workload": "decode B64 ctx~U[96,352] in a 4096-token block table, Hq32 Hkv8 D128 bf16, block_size 16, "
                        "20 calls per hipGraph replay",
            "tokens": tokens, "plan_part_tokens_parts_waves": list(paged_decode_plan(batch, hq, hkv, d, width // bs, bs)),
            "us_per_call": us16, "gbs": tokens * hkv * d * 4 / (us16 * 1e-6) / 1e9,
            "int8_us_per_call": us8, "int8_gbs": tokens * hkv * (2 * d + 8) / (us8 * 1e-6) / 1e9}


def bench_demo_shape(args):
    """The reference demo's attention shape (main.py:18-30: 16 query / 8 kv heads of 64 dims) in main.py's fp32 and
    in bf16: decode of 64 sequences of 1000-3000 tokens and prefill of 16 prompts of 64-2048 tokens."""
    import torch
    from helpers import make_paged_case_on_device, make_varlen_case
    from minivllm_amd.layers.attention import flash_attention_prefill, paged_attention_decode

    dev = "cuda:0"
    hq, hkv, d, bs = 16, 8, 64, 16
    out = {"workload": "Hq16 Hkv8 D64: decode B64 ctx~U[1000,3000] block_size 16; prefill 16 prompts L~U[64,2048]"}
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    flops = 4 * hq * d * sum(n * (n + 1) // 2 for n in lengths)
    for name, dtype in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        q, kc, vc, tables, ctx = make_paged_case_on_device(args.seed, dev, 64, 1000, 3000, hq, hkv, d, bs, dtype=dtype,
                                                           log_uniform=False)
        td, cd = tables.to(dev), ctx.to(dev)
        _, ms = time_steps(lambda: paged_attention_decode(q, kc, vc, td, cd, 1 / math.sqrt(d), hq, hkv, d, bs),
                           args.steps, args.warmup, EXTRA_WARM_MS)
        nbytes = int(ctx.sum()) * hkv * d * 2 * kc.element_size()
        out[f"decode_{name}_us"] = ms * 1e3
        out[f"decode_{name}_gbs"] = nbytes / (ms * 1e-3) / 1e9
        qq, kk, vv, cu = (t.to(dev) for t in make_varlen_case(args.seed + 1, lengths, hq, hkv, d, dtype=dtype))
        _, ms = time_steps(lambda: flash_attention_prefill(qq, kk, vv, cu, 1 / math.sqrt(d), hq, hkv, d),
                           args.steps, args.warmup, EXTRA_WARM_MS)
        out[f"prefill_{name}_ms"] = ms
        out[f"prefill_{name}_tflops"] = flops / (ms * 1e-3) / 1e12
    return out


def bench_other_head_dims(args):
    """bf16 head dims beside 64 and 128 that run on matrix-unit kernels (32, 80, 96, 112, 256: the decode kernels and
    the LDS-tiled prefill; 72: the same, with the first product's last step half empty) and one that does not (100: the generic
    kernels), on the demo leg's batch: decode of 64
    sequences of 1000-3000 tokens, prefill of 16 prompts of 64-2048 tokens, 16 query / 8 kv heads."""
    import torch
    from helpers import make_paged_case_on_device, make_varlen_case
    from minivllm_amd.layers.attention import flash_attention_prefill, paged_attention_decode, paged_decode_plan, prefill_plan

    dev = "cuda:0"
    hq, hkv, bs = 16, 8, 16
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(64, 2049, (16,), generator=g).tolist()
    out = {"workload": "bf16, Hq16 Hkv8: decode B64 ctx~U[1000,3000] block_size 16; prefill 16 prompts L~U[64,2048] "
                       f"(prefill timed after {EXTRA_WARM_MS:.0f} ms of warm-up launches, like the other prefill legs)"}
    for d in (32, 80, 96, 112, 256, 72, 100):
        q, kc, vc, tables, ctx = make_paged_case_on_device(args.seed, dev, 64, 1000, 3000, hq, hkv, d, bs,
                                                           dtype=torch.bfloat16, log_uniform=False)
        td, cd = tables.to(dev), ctx.to(dev)
        steps = args.steps if d != 100 else 3                      # the generic kernels are slow
        _, ms = time_steps(lambda: paged_attention_decode(q, kc, vc, td, cd, 1 / math.sqrt(d), hq, hkv, d, bs),
                           steps, min(args.warmup, steps), 0.0)
        nbytes = int(ctx.sum()) * hkv * d * 2 * kc.element_size()
        qq, kk, vv, cu = (t.to(dev) for t in make_varlen_case(args.seed + 1, lengths, hq, hkv, d, dtype=torch.bfloat16))
        _, pms = time_steps(lambda: flash_attention_prefill(qq, kk, vv, cu, 1 / math.sqrt(d), hq, hkv, d),
                            steps, min(args.warmup, steps), EXTRA_WARM_MS if d != 100 else 0.0)
        flops = 4 * hq * d * sum(n * (n + 1) // 2 for n in lengths)
        out[f"head_dim_{d}"] = {
            "decode_kernel": "generic" if paged_decode_plan(64, hq, hkv, d, tables.shape[1], bs, torch.bfloat16)[2] == 0 else "mfma",
            "decode_us": ms * 1e3, "decode_gbs": nbytes / (ms * 1e-3) / 1e9,
            "prefill_kernel": {0: "generic", 1: "16-row tiles", 2: "lds-tiled"}[prefill_plan(hq, hkv, d, dtype=torch.bfloat16)],
            "prefill_ms": pms, "prefill_tflops": flops / (pms * 1e-3) / 1e12,
        }
    return out


def bench_reference_shapes(args, want_cpu):
    """The shapes the reference's own benchmark scripts run (fp16, 32 query / 8 kv heads of 128 dims, block 16,
    identity block tables, every context the same length): decode (B, L) = (2,60) (1,512) (16,256) (4,2048)
    (benchmark_decoding.py:298-374) and prefill (seqs, L) = (2,60) (4,64) (2,1024) (1,4096)
    (benchmark_prefilling.py:427-495).  GPU time per call inside a hipGraph of 20 calls (these calls are latency,
    not bandwidth), the CPU oracle beside it (the PyTorch functions those scripts time, restated), and the
    difference between the two results."""
    import torch
    import oracle
    from minivllm_amd.layers.attention import flash_attention_prefill, paged_attention_decode

    dev = "cuda:0"
    hq, hkv, d, bs = 32, 8, 128, 16
    scale = 1.0 / math.sqrt(d)
    calls = 20

    def graph_us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(calls):
                fn()
        _, ms = time_steps(g.replay, args.steps, 2, EXTRA_WARM_MS)
        return ms * 1e3 / calls

    def cpu_ms(fn, budget_s=2.0):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            ref = fn()
            reps += 1
            if time.perf_counter() - t0 > budget_s or reps >= 50:
                return (time.perf_counter() - t0) / reps * 1e3, ref

    rows = {"decode": [], "prefill": []}
    gen = torch.Generator().manual_seed(args.seed)
    for batch, length in ((2, 60), (1, 512), (16, 256), (4, 2048)):
        mb = -(-length // bs)
        q = torch.randn(batch, hq, d, generator=gen).to(torch.float16)
        kc = torch.randn(batch * mb, bs, hkv, d, generator=gen).to(torch.float16)
        vc = torch.randn(batch * mb, bs, hkv, d, generator=gen).to(torch.float16)
        tables = torch.arange(batch * mb, dtype=torch.int32).reshape(batch, mb)
        ctx = torch.full((batch,), length, dtype=torch.int32)
        qd, kd, vd, td, cd = (t.to(dev) for t in (q, kc, vc, tables, ctx))
        us = graph_us(lambda: paged_attention_decode(qd, kd, vd, td, cd, scale, hq, hkv, d, bs))
        row = {"batch": batch, "context": length, "gpu_us_per_call": us}
        if want_cpu:
            got = paged_attention_decode(qd, kd, vd, td, cd, scale, hq, hkv, d, bs).float().cpu()
            args32 = (q.float(), kc.float(), vc.float(), tables, ctx, scale, hq, hkv, d, bs)
            row["cpu_naive_ms"], ref = cpu_ms(lambda: oracle.decode_naive_oracle(*args32))
            row["cpu_vectorised_ms"], _ = cpu_ms(lambda: oracle.decode_vectorised_oracle(*args32))
            row["gpu_vs_oracle_max_abs"] = (got - ref).abs().max().item()
        rows["decode"].append(row)
    for seqs, length in ((2, 60), (4, 64), (2, 1024), (1, 4096)):
        total = seqs * length
        q = torch.randn(total, hq, d, generator=gen).to(torch.float16)
        k = torch.randn(total, hkv, d, generator=gen).to(torch.float16)
        v = torch.randn(total, hkv, d, generator=gen).to(torch.float16)
        cu = torch.arange(seqs + 1, dtype=torch.int32) * length
        qd, kd, vd, cud = (t.to(dev) for t in (q, k, v, cu))
        us = graph_us(lambda: flash_attention_prefill(qd, kd, vd, cud, scale, hq, hkv, d))
        flops = 4 * hq * d * seqs * length * (length + 1) // 2
        row = {"seqs": seqs, "length": length, "gpu_us_per_call": us, "gpu_tflops": flops / (us * 1e-6) / 1e12}
        if want_cpu:
            got = flash_attention_prefill(qd, kd, vd, cud, scale, hq, hkv, d).float().cpu()
            row["cpu_standard_ms"], ref = cpu_ms(lambda: oracle.prefill_standard_oracle(q.float(), k.float(), v.float(), cu,
                                                                                        scale, hq, hkv, d))
            row["gpu_vs_oracle_max_abs"] = (got - ref).abs().max().item()
        rows["prefill"].append(row)
    rows["workload"] = ("the reference benchmark scripts' shapes: fp16, Hq32 Hkv8 D128, block_size 16, equal lengths; "
                        f"GPU: {calls} calls per hipGraph replay; CPU: the oracle (fp32) on {torch.get_num_threads()} threads")
    return rows


def bench_mfma_probe(args):
    """What the matrix unit sustains on this GPU (libmvllm_probe.so, csrc/mfma_probe.hip): register-only loops of
    v_mfma_f32_32x32x16_bf16 alone, with n v_fma_f32 (+ one v_exp_f32) issued after every MFMA by the same wave, and
    with the vector instructions on a second wave of the same SIMD.  The prefill tile body is 32 MFMAs and about 4
    other vector instructions + 1 exp per MFMA; these loops give its ceiling at the clock the GPU holds under that
    load.  Reported per mix: TFLOP/s of the MFMAs and the fraction of the 2.5 PFLOP/s data-sheet peak."""
    import ctypes
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "minivllm_amd", "libmvllm_probe.so"))
    fn = lib.mvllm_probe_mfma_mix
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int] * 5 + [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    out = torch.zeros(16, device="cuda:0")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    iters = 100000
    stream = torch.cuda.current_stream().cuda_stream

    def run(nv, ne, role, wps, per_cu=1):
        blocks = cus * per_cu

        def launch():
            st = fn(nv, ne, role, wps, blocks, out.data_ptr(), iters, stream)
            assert st == 0, st
        _, ms = time_steps(launch, 3, 1)
        torch.cuda.synchronize()
        clocks, ticks = out[1].item(), out[2].item()        # wave 0: shader clocks and 100 MHz ticks inside its loop
        mfma_waves = blocks * 4 * (1 if role == 1 else wps)
        flops = 0 if role == 2 else mfma_waves * iters * 4 * 32 * 32 * 16 * 2
        slots = blocks * 4 * wps * iters * 4 if role != 1 else blocks * 4 * iters * 4
        return {"ms": ms, "tflops": flops / (ms * 1e-3) / 1e12, "frac_of_peak": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                "shader_ghz": clocks / (ticks * 10.0) if ticks else None,
                # an MFMA alone is 32 clocks: 13.3 ns at 2.4 GHz
                "ns_per_slot_per_simd": ms * 1e6 / (slots / (cus * 4)),
                "clocks_per_slot_wave0": clocks / (iters * 4)}

    res = {"workload": f"register-only loops, {cus} CUs, {iters} iterations x 4 slots per wave; slot = 1 MFMA 32x32x16 bf16 + "
                       "nv v_fma_f32 + ne v_exp_f32", "mixes": {}}
    for wps in (1, 2):
        res["mixes"][f"mfma_only_{wps}wave_per_simd"] = run(0, 0, 0, wps)
    for chains, wps in ((1, 1), (2, 1), (1, 2), (2, 2)):      # fewer accumulator chains: an MFMA waits for the one before it
        res["mixes"][f"mfma_only_{chains}chain_{wps}wave_per_simd"] = run(100, chains, 0, wps)
    for nv, ne in ((2, 0), (4, 0), (6, 0), (8, 0), (0, 1), (3, 1), (4, 1)):
        res["mixes"][f"same_wave_nv{nv}_ne{ne}_2waves_per_simd"] = run(nv, ne, 0, 2)
    res["mixes"]["same_wave_nv4_ne1_1wave_per_simd"] = run(4, 1, 0, 1)
    for nv, ne in ((4, 0), (8, 0), (4, 1)):
        res["mixes"][f"other_wave_nv{nv}_ne{ne}"] = run(nv, ne, 1, 2)
        res["mixes"][f"vector_only_nv{nv}_ne{ne}_1wave_per_simd"] = run(nv, ne, 2, 1)
    return res


def bench_prefill_timeline(args):
    """Where a workgroup of the two-group prefill kernel spends a tile: the probe library's timing build logs the
    shader clock at the four corners of every tile (softmax begins / done, matrix part begins / done) for the waves of
    one workgroup.  A stamp costs about 100 clocks, so every logged interval is that much longer than in the product
    build; the shares are what the figures are for.  `workgroups`: from a second launch in which every workgroup logs
    only when it began and ended and what it went through (life in clocks; max over mean is what uneven dealing of
    the items costs)."""
    import ctypes
    import statistics
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "minivllm_amd", "libmvllm_probe.so"))
    fn = lib.mvllm_probe_prefill_timeline
    c = ctypes
    fn.restype = c.c_int
    fn.argtypes = [c.c_void_p] * 5 + [c.c_int, c.c_int64, c.c_int, c.c_int, c.c_int, c.c_float, c.c_int, c.c_void_p, c.c_int,
                   c.c_int, c.c_void_p]
    from minivllm_amd import _C
    dev = "cuda:0"
    hq, hkv, d = 32, 8, 128
    g = torch.Generator().manual_seed(args.seed)
    cfg2 = torch.randint(64, 2049, (16,), generator=g).tolist()
    out = {}
    for name, lengths in (("config2", cfg2), ("4x8192", [8192] * 4)):
        dg = torch.Generator(device=dev).manual_seed(args.seed + 1)
        total = sum(lengths)
        q, k, v = (torch.randn(total, h, d, generator=dg, device=dev).to(torch.bfloat16) for h in (hq, hkv, hkv))
        cu = torch.tensor([0] + lengths, dtype=torch.int32).cumsum(0).to(torch.int32).to(dev)
        o = torch.empty_like(q)
        entries = 2048
        log = torch.zeros(8, entries, dtype=torch.int64, device=dev)
        for _ in range(3):                                   # the last launch's stamps are read (clock settled)
            log.zero_()
            st = fn(o.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), cu.data_ptr(), len(lengths), total, hq, hkv, d,
                    1.0 / math.sqrt(d), _C.dtype_code(q.dtype), log.data_ptr(), entries, 9,
                    torch.cuda.current_stream().cuda_stream)
            assert st == 0, st
        torch.cuda.synchronize()
        rows = log.cpu().tolist()
        res = {"workgroup": 9, "note": "clocks; stamps at softmax begin, softmax done, matrix part begin, matrix part done"}
        for grp, wave in (("group0_wave0", 0), ("group1_wave4", 4)):
            t = [x for x in rows[wave] if x > 0]
            tiles = (len(t) - 1) // 4
            seg = [[t[4 * i + j + 1] - t[4 * i + j] for i in range(tiles)] for j in range(4)]
            per_tile = [t[4 * i + 4] - t[4 * i] for i in range(tiles)]
            med = lambda xs: int(statistics.median(xs)) if xs else None
            res[grp] = {"tiles_logged": tiles, "softmax": med(seg[0]), "wait_for_matrix_part": med(seg[1]),
                        "matrix_part": med(seg[2]), "wait_for_softmax": med(seg[3]), "tile": med(per_tile),
                        "life": t[-1] - t[0] if t else None}
        # every workgroup's begin and end (block < 0): how evenly the items were dealt
        grid = torch.cuda.get_device_properties(0).multi_processor_count // 8 * 8
        per_wg = torch.zeros(grid, 4, dtype=torch.int64, device=dev)
        for _ in range(3):
            per_wg.zero_()
            st = fn(o.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), cu.data_ptr(), len(lengths), total, hq, hkv, d,
                    1.0 / math.sqrt(d), _C.dtype_code(q.dtype), per_wg.data_ptr(), 4, -1,
                    torch.cuda.current_stream().cuda_stream)
            assert st == 0, st
        torch.cuda.synchronize()
        rows = [r for r in per_wg.cpu().tolist() if r[1] > r[0]]
        life = [r[1] - r[0] for r in rows]
        res["workgroups"] = {"busy": len(rows), "life_max": max(life), "life_mean": int(sum(life) / len(life)),
                             "max_over_mean": round(max(life) * len(life) / sum(life), 4),
                             "items_max": max(r[2] for r in rows), "items_min": min(r[2] for r in rows),
                             "tiles_max": max(r[3] for r in rows), "tiles_mean": round(sum(r[3] for r in rows) / len(rows), 2)}
        out[name] = res
    return out


def bench_engine(args, max_num_sequences, graph):
    """BASELINE.json config 5: random-init Qwen3-style decoder (hidden 1024, 8 layers, Hq16/Hkv8/D128, FFN 3072,
    vocab 151936, bf16), 60 prompts of random ids with lengths U[32,96], 256 new tokens each, T 0.6."""
    import torch
    from minivllm_amd.engine.llm_engine import LLMEngine
    from minivllm_amd.sampling_parameters import SamplingParams

    cfg = dict(vocab_size=151936, hidden_size=1024, num_layers=8, num_heads=16, num_kv_heads=8, head_dim=128,
               intermediate_size=3072, base=1_000_000, rms_norm_epsilon=1e-6, qkv_bias=False, ffn_bias=True,
               scale=1.0, tie_word_embeddings=True, block_size=256, max_num_batched_tokens=16384,
               max_num_sequences=max_num_sequences, max_cached_blocks=256, max_position=512,
               max_model_length=512, enforce_eager=not graph, dtype="bf16", eos=-1, seed=args.seed)
    g = torch.Generator().manual_seed(args.seed)
    lengths = torch.randint(32, 97, (60,), generator=g).tolist()
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]
    engine = LLMEngine(cfg)
    sp = SamplingParams(temperature=0.6, max_tokens=256, ignore_eos=True)
    engine.generate(prompts[:4], SamplingParams(temperature=0.6, max_tokens=4, ignore_eos=True))   # warm-up
    for key in engine.stats:
        engine.stats[key] = 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = engine.generate(prompts, sp)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    new_tokens = sum(len(t) for t in out["token_ids"])
    assert new_tokens == 60 * 256
    return {
        "workload": "engine generate: 60 prompts L~U[32,96], 256 new tokens each, Qwen3-style 8x1024 bf16, "
                    f"block_size 256, max_num_sequences {max_num_sequences}, "
                    + ("hipGraph decode" if graph else "eager decode"),
        "output_tokens": new_tokens, "wall_s": wall, "tok_per_s": new_tokens / wall,
        "steps": engine.stats["steps"], "decode_s": engine.stats["decode_s"], "prefill_s": engine.stats["prefill_s"],
    }


def summary_of(line):
    """The figures of every quantity the metric names, in a few hundred characters, for the end of the JSON line."""
    ex = line["extra"]
    r3 = lambda x: None if x is None else round(x, 3)
    out = {"decode_frac_hbm": r3(line["roofline"]["frac"]), "decode_gbs": round(line["roofline"]["achieved"])}
    def put(key, leg, *path):
        node = ex.get(leg)
        for p_ in path:
            node = node.get(p_) if isinstance(node, dict) else None
        if node is not None:
            out[key] = r3(node) if isinstance(node, float) else node
    b256 = ex.get("decode_block256")
    if isinstance(b256, dict) and "gbs_event" in b256:
        out["decode_bs256_frac_hbm"] = r3(b256["gbs_event"] / HBM_PEAK_GBS)
    put("prefill_frac_mfma", "prefill", "roofline", "frac")
    put("prefill_tflops", "prefill", "tflops")
    put("prefill_us", "prefill", "event_ms_per_step")
    put("prefill_vs_oracle_max_abs", "prefill", "cpu_baseline", "gpu_vs_oracle_max_abs")
    put("prefill_hq16_frac", "prefill_hq16", "roofline", "frac")
    put("prefill_4x8192_frac", "prefill_long_prompts", "roofline", "frac")
    put("prefill_suffix128_behind_32k_us", "prefill_short_suffix", "event_ms_per_step")
    put("prefill_paged_frac", "prefill_cached_prefix", "roofline", "frac")
    put("prefill_paged_int8_frac", "prefill_cached_prefix_int8", "roofline", "frac")
    put("prefill_d256_tflops", "other_head_dims", "head_dim_256", "prefill_tflops")
    put("prefill_d96_tflops", "other_head_dims", "head_dim_96", "prefill_tflops")
    put("store_frac_hbm", "store", "roofline", "frac")
    put("int8_decode_frac_hbm", "int8", "roofline", "frac")
    put("int8_store_frac_hbm", "int8", "store_roofline", "frac")
    put("int8_decode_vs_oracle_max_abs", "int8", "gpu_vs_oracle_max_abs")
    for key, leg in (("engine16_eager_tok_s", "engine_16seq_eager"), ("engine16_tok_s", "engine_16seq_graph"), ("engine64_tok_s", "engine_64seq_graph")):
        node = ex.get(leg)
        if isinstance(node, dict):
            for name in ("out_tok_per_s", "tok_per_s", "output_tokens_per_s"):
                if name in node:
                    out[key] = round(node[name])
                    break
    for key in ("prefill_d256_tflops", "prefill_d96_tflops"):
        if key in out:
            out[key] = round(out[key])
    for key in ("prefill_us", "prefill_suffix128_behind_32k_us"):
        if key in out:
            out[key] = round(out[key] * 1e3, 1)
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives or sharding are part of it); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    from minivllm_amd import _C
    _C.load()

    if args.calib_copy:
        src = torch.ones(1 << 30, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    only = set(x for x in args.only.split(",") if x)
    want = lambda name: not only or name in only
    extra = {}
    head, cpu = bench_decode(args, args.block_size, want_cpu=not args.no_cpu and want("cpu"),
                             want_probe=want("loads_probe"))
    if want("decode256") and args.block_size != 256:
        extra["decode_block256"], _ = bench_decode(args, 256, want_cpu=False)
    want_cpu = not args.no_cpu and want("cpu")
    which = [n for n in ("prefill", "prefill_long", "store") if want(n)]
    if which:
        extra.update(bench_prefill_store(args, which, want_cpu))
    if want("int8"):
        extra["int8"] = bench_int8(args, want_cpu, want("loads_probe"))
    if want("reference_shapes"):
        extra["reference_benchmark_shapes"] = bench_reference_shapes(args, want_cpu)
    if want("decode_small"):
        extra["decode_small_batch"] = bench_decode_small(args)
    if want("demo_shape"):
        extra["reference_demo_shape"] = bench_demo_shape(args)
    if want("head_dims"):
        extra["other_head_dims"] = bench_other_head_dims(args)
    if want("fused_qk"):
        extra["fused_qk"] = bench_fused_qk(args)
    if want("sampler"):
        extra["sampler"] = bench_sampler(args)
    if want("mfma_probe"):
        extra["mfma_probe"] = bench_mfma_probe(args)
    if want("prefill_timeline"):
        extra["prefill_timeline"] = bench_prefill_timeline(args)
    if want("engine"):
        extra["engine_16seq_eager"] = bench_engine(args, 16, False)
        extra["engine_16seq_graph"] = bench_engine(args, 16, True)
        extra["engine_64seq_graph"] = bench_engine(args, 64, True)
    else:                                              # one configuration alone, as a kernel trace of a decode step wants
        if "engine16" in only:
            extra["engine_16seq_graph"] = bench_engine(args, 16, True)
        if "engine64" in only:
            extra["engine_64seq_graph"] = bench_engine(args, 64, True)

    if "loads_only" in head:
        extra["decode_loads_only"] = head["loads_only"]
    line = {
        "metric": "decode-attn HBM GB/s (% peak); prefill TFLOP/s (% MFMA); engine out tok/s",
        "value": head["gbs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seeded N(0,1) q/K/V, random disjoint block tables, seed %d)" % args.seed,
        "config": {"workload": head["workload"], "tokens": head["tokens"], "algorithmic_bytes": head["algorithmic_bytes"]},
        "roofline": {
            "bound": "hbm",
            "achieved": head["gbs_event"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": head["gbs_event"] / HBM_PEAK_GBS,
            "traffic": DECODE_TRAFFIC_BYTES_DEFAULT if (args.seed == 0 and args.block_size == 16) else None,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload summarised in "
                              "profiles/bench_hbm_traffic_pmc.txt (a counter run cannot time; not re-measured in this run)",
            "kernel": "decode_mfma_kernel + decode_reduce_vec_kernel (one decode call, HIP events on the launch stream)",
        },
        "cpu_baseline": cpu,
        "extra": extra,
    }
    line["summary"] = summary_of(line)     # last on purpose: a record that keeps only the end of the line keeps this
    print(json.dumps(line))


if __name__ == "__main__":
    main()
