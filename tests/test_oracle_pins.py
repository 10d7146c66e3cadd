"""Pins the CPU oracle against what the mathematics fixes (the reference has no
tests, golden vectors or fixtures for this path).  Each check is chosen so a
plausible slip (dropped scale, wrong GQA map, off-by-one in the causal mask or
block arithmetic, transposed operand) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import make_paged_case, make_slot_mapping, make_varlen_case


# ---------------------------------------------------------------- store -----
def test_store_closed_form_on_poisoned_cache():
    lengths = [5, 33, 16]
    bs, hkv, d = 16, 2, 8
    slots, _, nb = make_slot_mapping(1, lengths, bs)
    t = sum(lengths)
    g = torch.Generator().manual_seed(2)
    key = torch.randn(t, hkv, d, generator=g)
    val = torch.randn(t, hkv, d, generator=g)
    slots[7] = -1                                    # a skipped token
    kc = torch.full((nb, bs, hkv, d), 777.0)
    vc = torch.full((nb, bs, hkv, d), -777.0)
    oracle.store_kvcache_oracle(key, val, kc, vc, slots, bs)
    flat_k, flat_v = kc.view(-1, hkv, d), vc.view(-1, hkv, d)
    written = torch.zeros(nb * bs, dtype=torch.bool)
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        written[s] = True
        assert torch.equal(flat_k[s], key[i]) and torch.equal(flat_v[s], val[i])
    assert (flat_k[~written] == 777.0).all() and (flat_v[~written] == -777.0).all()
    assert written.sum().item() == t - 1


def test_store_round_trip_through_block_table():
    """Store with engine-style slots, gather back by block table: identity."""
    lengths = [40, 7]
    bs, hkv, d = 16, 2, 4
    slots, tables, nb = make_slot_mapping(3, lengths, bs)
    g = torch.Generator().manual_seed(4)
    key = torch.randn(sum(lengths), hkv, d, generator=g)
    val = torch.randn(sum(lengths), hkv, d, generator=g)
    kc = torch.zeros(nb, bs, hkv, d)
    vc = torch.zeros(nb, bs, hkv, d)
    oracle.store_kvcache_oracle(key, val, kc, vc, slots, bs)
    at = 0
    for n, blocks in zip(lengths, tables):
        row = torch.tensor(blocks, dtype=torch.int32)
        assert torch.equal(oracle.gather_sequence_kv(kc, row, n, bs), key[at:at + n])
        assert torch.equal(oracle.gather_sequence_kv(vc, row, n, bs), val[at:at + n])
        at += n


# --------------------------------------------------------------- decode -----
def _brute_force_decode(q, kc, vc, tables, ctx, scale, hq, hkv, bs):
    out = torch.zeros(q.shape, dtype=torch.float64)
    rep = hq // hkv
    for b in range(q.shape[0]):
        for h in range(hq):
            g = h // rep
            scores, rows = [], []
            for t in range(int(ctx[b])):
                blk = int(tables[b, t // bs])
                kvec = kc[blk, t % bs, g].double()
                scores.append(float((q[b, h].double() * kvec).sum()) * scale)
                rows.append(vc[blk, t % bs, g].double())
            mx = max(scores)
            w = [math.exp(s - mx) for s in scores]
            tot = sum(w)
            for wi, r in zip(w, rows):
                out[b, h] += (wi / tot) * r
    return out


@pytest.mark.parametrize("fn", [oracle.decode_naive_oracle, oracle.decode_vectorised_oracle])
def test_decode_matches_fp64_brute_force(fn):
    hq, hkv, d, bs = 4, 2, 8, 4
    q, kc, vc, tables, ctx = make_paged_case(5, 3, 1, 19, hq, hkv, d, bs)
    scale = 0.37
    got = fn(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
    want = _brute_force_decode(q, kc, vc, tables, ctx, scale, hq, hkv, bs)
    assert torch.allclose(got.double(), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("fn", [oracle.decode_naive_oracle, oracle.decode_vectorised_oracle])
def test_decode_special_cases(fn):
    hq, hkv, d, bs = 4, 2, 8, 4
    # ctx = 1 -> output is V[token 0] of the shared kv head, whatever q and scale are
    q, kc, vc, tables, ctx = make_paged_case(6, 2, 1, 1, hq, hkv, d, bs)
    got = fn(q, kc, vc, tables, ctx, 3.0, hq, hkv, d, bs)
    for b in range(2):
        for h in range(hq):
            assert torch.allclose(got[b, h], vc[int(tables[b, 0]), 0, h // 2], atol=1e-6)
    # all K rows equal -> uniform mean of the V rows
    q, kc, vc, tables, ctx = make_paged_case(7, 2, 5, 11, hq, hkv, d, bs)
    kc[:] = kc[0, 0, 0]
    got = fn(q, kc, vc, tables, ctx, 1.0, hq, hkv, d, bs)
    for b in range(2):
        n = int(ctx[b])
        rows = oracle.gather_sequence_kv(vc, tables[b], n, bs)
        for h in range(hq):
            assert torch.allclose(got[b, h], rows[:, h // 2].mean(0), atol=1e-5)


def test_decode_identity_table_equals_dense_sdpa():
    hq, hkv, d, bs, n = 4, 2, 16, 8, 24
    g = torch.Generator().manual_seed(8)
    q = torch.randn(2, hq, d, generator=g)
    kc = torch.randn(6, bs, hkv, d, generator=g)
    vc = torch.randn(6, bs, hkv, d, generator=g)
    tables = torch.arange(6, dtype=torch.int32).reshape(2, 3)
    ctx = torch.tensor([n, n])
    scale = 1 / math.sqrt(d)
    got = oracle.decode_naive_oracle(q, kc, vc, tables, ctx, scale, hq, hkv, d, bs)
    kd = kc.reshape(2, n, hkv, d).repeat_interleave(2, dim=2).transpose(1, 2)
    vd = vc.reshape(2, n, hkv, d).repeat_interleave(2, dim=2).transpose(1, 2)
    want = F.scaled_dot_product_attention(q.unsqueeze(2), kd, vd, scale=scale).squeeze(2)
    assert torch.allclose(got, want, atol=1e-5)


def test_decode_block_permutation_invariance_and_agreement():
    hq, hkv, d, bs = 8, 2, 16, 4
    q, kc, vc, tables, ctx = make_paged_case(9, 4, 3, 30, hq, hkv, d, bs)
    a = oracle.decode_naive_oracle(q, kc, vc, tables, ctx, 0.25, hq, hkv, d, bs)
    b = oracle.decode_vectorised_oracle(q, kc, vc, tables, ctx, 0.25, hq, hkv, d, bs)
    assert torch.allclose(a, b, atol=1e-6)
    perm = torch.randperm(kc.shape[0], generator=torch.Generator().manual_seed(10))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    kc2, vc2 = kc[perm], vc[perm]                      # new block j holds old block perm[j]
    tables2 = torch.where(tables >= 0, inv[tables.clamp(min=0).long()].to(torch.int32), tables)
    c = oracle.decode_naive_oracle(q, kc2, vc2, tables2, ctx, 0.25, hq, hkv, d, bs)
    assert torch.equal(a, c)


# -------------------------------------------------------------- prefill -----
def test_prefill_matches_library_sdpa_and_row0():
    hq, hkv, d = 4, 2, 16
    lengths = [1, 7, 33, 12]
    q, k, v, cu = make_varlen_case(11, lengths, hq, hkv, d)
    scale = 1 / math.sqrt(d)
    got = oracle.prefill_standard_oracle(q, k, v, cu, scale, hq, hkv, d)
    at = 0
    for n in lengths:
        qs = q[at:at + n].transpose(0, 1).unsqueeze(0)
        ks = k[at:at + n].transpose(0, 1).repeat_interleave(2, dim=0).unsqueeze(0)
        vs = v[at:at + n].transpose(0, 1).repeat_interleave(2, dim=0).unsqueeze(0)
        want = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, scale=scale)[0].transpose(0, 1)
        assert torch.allclose(got[at:at + n], want, atol=1e-5)
        # first row of a sequence sees only itself
        for h in range(hq):
            assert torch.allclose(got[at, h], v[at, h // 2], atol=1e-6)
        at += n


def test_prefill_fp64_brute_force_and_independence():
    hq, hkv, d = 2, 1, 4
    lengths = [3, 5]
    q, k, v, cu = make_varlen_case(12, lengths, hq, hkv, d)
    scale = 0.8
    got = oracle.prefill_standard_oracle(q, k, v, cu, scale, hq, hkv, d)
    at = 0
    for n in lengths:
        for i in range(n):
            for h in range(hq):
                s = [float((q[at + i, h].double() * k[at + j, 0].double()).sum()) * scale for j in range(i + 1)]
                mx = max(s)
                w = [math.exp(x - mx) for x in s]
                want = sum(wj * v[at + j, 0].double() for j, wj in enumerate(w)) / sum(w)
                assert torch.allclose(got[at + i, h].double(), want, atol=1e-6)
        at += n
    # changing the second prompt leaves the first prompt's rows bit-identical
    k2, v2 = k.clone(), v.clone()
    k2[3:] += 1.0
    v2[3:] -= 2.0
    got2 = oracle.prefill_standard_oracle(q, k2, v2, cu, scale, hq, hkv, d)
    assert torch.equal(got[:3], got2[:3])


def test_prefill_last_row_equals_decode_after_store():
    hq, hkv, d, bs = 4, 2, 8, 4
    lengths = [9, 4]
    q, k, v, cu = make_varlen_case(13, lengths, hq, hkv, d)
    slots, tables, nb = make_slot_mapping(14, lengths, bs)
    kc = torch.zeros(nb, bs, hkv, d)
    vc = torch.zeros(nb, bs, hkv, d)
    oracle.store_kvcache_oracle(k, v, kc, vc, slots, bs)
    width = max(len(t) for t in tables)
    bt = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32)
    last = torch.tensor([8, 12])
    pre = oracle.prefill_standard_oracle(q, k, v, cu, 0.5, hq, hkv, d)
    dec = oracle.decode_naive_oracle(q[last], kc, vc, bt, torch.tensor(lengths), 0.5, hq, hkv, d, bs)
    assert torch.allclose(pre[last], dec, atol=1e-6)


# ----------------------------------------------------------------- int8 -----
def test_int8_spec_invariants():
    g = torch.Generator().manual_seed(15)
    x = torch.randn(64, 4, 128, generator=g)
    x[torch.rand(x.shape, generator=g) < 0.01] *= 8.0
    x[3, 1] = 0.0                                      # an all-zero vector
    codes, scale = oracle.quantize_int8_oracle(x)
    assert codes.dtype == torch.int8 and scale.dtype == torch.float32
    amax = x.abs().amax(-1)
    assert torch.equal(scale, amax / torch.tensor(127.0))          # bit-equal fp32 division
    assert codes.abs().max().item() <= 127
    live = amax > 0
    assert (codes.abs().amax(-1)[live] == 127).all()               # the absmax element maps to +-127
    assert (codes[3, 1] == 0).all() and scale[3, 1] == 0
    err = (x - codes.float() * scale.unsqueeze(-1)).abs()
    assert (err <= scale.unsqueeze(-1) * 0.5 * (1 + 1e-5)).all()
    # sign symmetry and round-half-even on exact ties
    c2, s2 = oracle.quantize_int8_oracle(-x)
    assert torch.equal(c2, -codes) and torch.equal(s2, scale)
    t = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 3.49, 0.0]])
    ct, st = oracle.quantize_int8_oracle(t)
    assert st.item() == 1.0 and ct.tolist() == [[127, 0, 2, 2, 0, -2, 3, 0]]


def test_int8_store_then_decode_close_to_fp32():
    hq, hkv, d, bs = 4, 2, 32, 4
    lengths = [13, 6]
    g = torch.Generator().manual_seed(16)
    k = torch.randn(sum(lengths), hkv, d, generator=g)
    v = torch.randn(sum(lengths), hkv, d, generator=g)
    slots, tables, nb = make_slot_mapping(17, lengths, bs)
    kc = torch.zeros(nb, bs, hkv, d, dtype=torch.int8)
    vc = torch.zeros_like(kc)
    ks = torch.zeros(nb, bs, hkv)
    vs = torch.zeros_like(ks)
    oracle.store_kvcache_int8_oracle(k, v, kc, vc, ks, vs, slots, bs)
    kf = torch.zeros(nb, bs, hkv, d)
    vf = torch.zeros_like(kf)
    oracle.store_kvcache_oracle(k, v, kf, vf, slots, bs)
    width = max(len(t) for t in tables)
    bt = torch.tensor([t + [-1] * (width - len(t)) for t in tables], dtype=torch.int32)
    q = torch.randn(2, hq, d, generator=g)
    ctx = torch.tensor(lengths)
    a = oracle.decode_int8_oracle(q, kc, vc, ks, vs, bt, ctx, 0.2, hq, hkv, d, bs)
    b = oracle.decode_naive_oracle(q, kf, vf, bt, ctx, 0.2, hq, hkv, d, bs)
    assert (a - b).abs().max().item() < 0.05
    assert torch.equal(oracle.dequantize_cache_oracle(kc, ks).view(-1, hkv, d)[slots],
                       oracle.quantize_int8_oracle(k)[0].float() * oracle.quantize_int8_oracle(k)[1].unsqueeze(-1))


# ------------------------------------------------------------ producers -----
def test_prefill_metadata_reference_example():
    """model_runner.py:174-179: three prompts of 3, 2, 4 tokens -> cu_seqlens_q [0,3,5,9]."""
    bs = 4
    seqs = [dict(num_tokens=3, num_cached_tokens=0, block_table=[5]),
            dict(num_tokens=2, num_cached_tokens=0, block_table=[2]),
            dict(num_tokens=4, num_cached_tokens=0, block_table=[7])]
    md = oracle.prefill_metadata_oracle(seqs, bs)
    assert md["cu_seqlens_q"] == [0, 3, 5, 9] and md["cu_seqlens_k"] == [0, 3, 5, 9]
    assert md["slot_mapping"] == [20, 21, 22, 8, 9, 28, 29, 30, 31]
    assert md["max_seqlen_q"] == 4 and md["block_tables"] is None


def test_prefill_metadata_with_cached_prefix():
    bs = 4
    seqs = [dict(num_tokens=10, num_cached_tokens=4, block_table=[3, 9, 1]),
            dict(num_tokens=2, num_cached_tokens=0, block_table=[6])]
    md = oracle.prefill_metadata_oracle(seqs, bs)
    assert md["cu_seqlens_q"] == [0, 6, 8] and md["cu_seqlens_k"] == [0, 10, 12]
    assert md["slot_mapping"] == [36, 37, 38, 39, 4, 5, 24, 25]
    assert md["block_tables"] == [[3, 9, 1], [6, -1, -1]]
    assert md["token_ranges"] == [(4, 10), (0, 2)]


def test_decode_metadata_hand_worked():
    bs = 4
    seqs = [dict(num_tokens=5, block_table=[2, 8], last_token=11),     # 5th token -> block 8 offset 0
            dict(num_tokens=4, block_table=[3], last_token=12),        # exact multiple -> block 3 offset 3
            dict(num_tokens=11, block_table=[0, 1, 7], last_token=13)]
    md = oracle.decode_metadata_oracle(seqs, bs)
    assert md["slot_mapping"] == [32, 15, 30]
    assert md["context_lens"] == [5, 4, 11] and md["input_ids"] == [11, 12, 13]
    assert md["block_tables"] == [[2, 8, -1], [3, -1, -1], [0, 1, 7]]


def test_metadata_slots_unique_and_owned():
    from hypothesis import given, settings, strategies as st

    @settings(max_examples=200, deadline=None, derandomize=True)
    @given(st.lists(st.integers(1, 70), min_size=1, max_size=6), st.sampled_from([1, 4, 16]))
    def run(lengths, bs):
        at, seqs = 0, []
        for n in lengths:
            nb = -(-n // bs)
            seqs.append(dict(num_tokens=n, num_cached_tokens=0, block_table=list(range(at, at + nb)),
                             last_token=0))
            at += nb
        md = oracle.prefill_metadata_oracle(seqs, bs)
        slots = md["slot_mapping"]
        assert len(slots) == sum(lengths) == md["cu_seqlens_q"][-1]
        assert len(set(slots)) == len(slots)
        pos = 0
        for s in seqs:
            for i in range(s["num_tokens"]):
                assert slots[pos] == s["block_table"][i // bs] * bs + i % bs
                pos += 1
        dm = oracle.decode_metadata_oracle(seqs, bs)
        for s, slot in zip(seqs, dm["slot_mapping"]):
            n = s["num_tokens"]
            assert slot == s["block_table"][(n - 1) // bs] * bs + (n - 1) % bs

    run()


# ---------------------------------------------------------------------------
# caller-side chain: RMSNorm, rotary table, rotation (layernorm.py:9-17, rotary_embedding.py:4-83)
# ---------------------------------------------------------------------------
def test_rms_norm_oracle_closed_forms():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(7, 3, 64, generator=g)
    ones = torch.ones(64)
    y = oracle.rms_norm_oracle(x, ones, 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(7, 3), atol=1e-5)          # unit mean square
    assert torch.allclose(oracle.rms_norm_oracle(3.5 * x, ones, 0.0), y, atol=1e-5)  # scale invariant at eps 0
    c = torch.full((1, 1, 64), -2.0)
    gamma = torch.linspace(0.5, 2.0, 64)
    want = -2.0 / math.sqrt(4.0 + 0.25) * gamma                                    # constant vector, eps 0.25
    assert torch.allclose(oracle.rms_norm_oracle(c, gamma, 0.25)[0, 0], want, atol=1e-6)
    big_eps = oracle.rms_norm_oracle(x, ones, 1e6)                                 # eps sits inside the root
    assert torch.allclose(big_eps, x / math.sqrt(1e6), rtol=1e-3, atol=1e-7)


def test_rope_table_matches_fp64_formula():
    base, d, n = 10000.0, 32, 50
    table = oracle.rope_cos_sin_cache_oracle(base, d, n)
    assert table.shape == (n, d) and table.dtype == torch.float32
    pos = torch.arange(n, dtype=torch.float64).unsqueeze(1)
    inv = torch.tensor([base ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64).unsqueeze(0)
    assert torch.allclose(table[:, : d // 2].double(), torch.cos(pos * inv), atol=2e-5)
    assert torch.allclose(table[:, d // 2:].double(), torch.sin(pos * inv), atol=2e-5)


def test_rope_oracle_sign_pairing_and_group_law():
    d = 8
    table = oracle.rope_cos_sin_cache_oracle(10000.0, d, 64)
    # position 0 is the identity
    g = torch.Generator().manual_seed(9)
    x = torch.randn(5, 2, d, generator=g)
    assert torch.equal(oracle.rope_oracle(x, torch.zeros(5, dtype=torch.long), table), x)
    # hand-worked: inv_freq[0] = 1, so at position 1 the unit vector e_0 turns by +1 rad in the (0, d/2) plane
    e0 = torch.zeros(1, 1, d); e0[0, 0, 0] = 1.0
    y = oracle.rope_oracle(e0, torch.tensor([1]), table)[0, 0]
    want = torch.zeros(d); want[0] = math.cos(1.0); want[d // 2] = math.sin(1.0)
    assert torch.allclose(y, want, atol=1e-6)
    # e_{d/2} turns to (-sin, cos): the sign of the second row of the rotation
    e4 = torch.zeros(1, 1, d); e4[0, 0, d // 2] = 1.0
    y = oracle.rope_oracle(e4, torch.tensor([1]), table)[0, 0]
    want = torch.zeros(d); want[0] = -math.sin(1.0); want[d // 2] = math.cos(1.0)
    assert torch.allclose(y, want, atol=1e-6)
    # every (i, i + d/2) pair keeps its norm, nothing leaks between pairs
    pos = torch.tensor([3, 17, 40, 63, 1])
    y = oracle.rope_oracle(x, pos, table)
    n_in = x[..., : d // 2] ** 2 + x[..., d // 2:] ** 2
    n_out = y[..., : d // 2] ** 2 + y[..., d // 2:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-5)
    # angles add: rotating to position a and then by b more equals rotating to a + b
    a, b = torch.tensor([5] * 5), torch.tensor([9] * 5)
    assert torch.allclose(oracle.rope_oracle(oracle.rope_oracle(x, a, table), b, table),
                          oracle.rope_oracle(x, a + b, table), atol=1e-5)
    # scores depend on the position difference only
    q, k = torch.randn(1, 1, d, generator=g), torch.randn(1, 1, d, generator=g)
    s1 = (oracle.rope_oracle(q, torch.tensor([20]), table) * oracle.rope_oracle(k, torch.tensor([13]), table)).sum()
    s2 = (oracle.rope_oracle(q, torch.tensor([47]), table) * oracle.rope_oracle(k, torch.tensor([40]), table)).sum()
    assert abs(float(s1 - s2)) < 1e-4


def test_fused_chain_oracle_is_the_composition():
    g = torch.Generator().manual_seed(11)
    t, hq, hkv, d, bs = 9, 4, 2, 16, 4
    q, k, v = (torch.randn(t, h, d, generator=g).to(torch.bfloat16) for h in (hq, hkv, hkv))
    table = oracle.rope_cos_sin_cache_oracle(1e6, d, 32)
    pos = torch.randint(0, 32, (t,), generator=g)
    gamma = torch.rand(d, generator=g) + 0.5
    slots = torch.tensor([0, 1, 2, -1, 8, 9, 10, 11, 5])
    kc = torch.zeros(3, bs, hkv, d, dtype=torch.bfloat16); vc = torch.zeros_like(kc)
    q_out, k_out = oracle.qk_norm_rope_store_oracle(q, k, v, pos, table, gamma, 1e-6, slots, kc, vc, block_size=bs)
    assert torch.equal(q_out, oracle.rope_oracle(oracle.rms_norm_oracle(q, gamma, 1e-6), pos, table))
    flat = kc.view(-1, hkv, d)
    assert torch.equal(flat[8], k_out[4]) and torch.equal(flat[5], k_out[8])
    assert torch.equal(vc.view(-1, hkv, d)[2], v[2])
    assert float(flat[3].abs().sum()) == 0.0                                        # slot 3 never written (token 3 skipped)
    # no gamma: rotation only
    q2, _ = oracle.qk_norm_rope_store_oracle(q, k, v, pos, table, None, 1e-6)
    assert torch.equal(q2, oracle.rope_oracle(q, pos, table))


# ---------------------------------------------------------------------------
# prefill after a cached prefix (metadata of model_runner.py:192-226)
# ---------------------------------------------------------------------------
def test_prefill_paged_oracle_is_the_tail_of_a_full_prefill():
    from helpers import make_paged_prefill_case
    hq, hkv, d, bs = 4, 2, 16, 8
    lengths, cached = [37, 8, 50, 19], [16, 0, 49, 8]
    c = make_paged_prefill_case(31, lengths, cached, hq, hkv, d, bs)
    scale = 1.0 / math.sqrt(d)
    full = oracle.prefill_standard_oracle(c["q"], c["k"], c["v"], c["cu_k"], scale, hq, hkv, d)
    got = oracle.prefill_paged_oracle(c["q_new"], c["k_cache"], c["v_cache"], c["block_tables"], c["cu_q"],
                                      c["cu_k"], scale, hq, hkv, d, bs)
    assert torch.allclose(got, full[c["new_rows"]], atol=1e-5)
    # no cached prefix anywhere: it is the plain prefill
    c0 = make_paged_prefill_case(32, lengths, [0] * 4, hq, hkv, d, bs)
    got0 = oracle.prefill_paged_oracle(c0["q_new"], c0["k_cache"], c0["v_cache"], c0["block_tables"], c0["cu_q"],
                                       c0["cu_k"], scale, hq, hkv, d, bs)
    want0 = oracle.prefill_standard_oracle(c0["q"], c0["k"], c0["v"], c0["cu_k"], scale, hq, hkv, d)
    assert torch.allclose(got0, want0, atol=1e-5)
    # exactly one new token per sequence: it is a decode step over the same cache
    c1 = make_paged_prefill_case(33, lengths, [n - 1 for n in lengths], hq, hkv, d, bs)
    got1 = oracle.prefill_paged_oracle(c1["q_new"], c1["k_cache"], c1["v_cache"], c1["block_tables"], c1["cu_q"],
                                       c1["cu_k"], scale, hq, hkv, d, bs)
    kc = torch.nan_to_num(c1["k_cache"], nan=0.0)      # the decode oracle pads with whole blocks
    vc = torch.nan_to_num(c1["v_cache"], nan=0.0)
    dec = oracle.decode_naive_oracle(c1["q_new"], kc, vc, c1["block_tables"], torch.tensor(lengths), scale,
                                     hq, hkv, d, bs)
    assert torch.allclose(got1, dec, atol=1e-5)


# ---------------------------------------------------------------------------
# sampler (sampler.py:14-19) and the counter-based noise of the HIP sampler
# ---------------------------------------------------------------------------
def test_philox_known_answer_vectors():
    """Philox4x32-10 vectors published with the Random123 library (kat_vectors)."""
    import numpy as np
    kat = [
        ([0, 0, 0, 0], (0, 0), "6627e8d5 e169c58d bc57ac4c 9b00dbd8"),
        ([0xffffffff] * 4, (0xffffffff, 0xffffffff), "408f276d 41c83b0e a20bc7c6 6d5451fd"),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], (0xa4093822, 0x299f31d0),
         "d16cfe09 94fdcceb 5001e420 24126ea1"),
    ]
    for ctr, key, want in kat:
        got = oracle.philox4x32_10_oracle(np.array([ctr], dtype=np.uint32), key)[0]
        assert " ".join("%08x" % int(x) for x in got) == want


def test_exponential_noise_is_exponential_and_counter_addressed():
    e = oracle.exponential_noise_oracle(seed=7, offset=3, batch=4, vocab=50001)
    assert e.shape == (4, 50001) and e.dtype == torch.float32
    assert float(e.min()) > 0 and float(e.max()) < 17.4               # u in (2^-25, 1 - 2^-25)
    assert abs(float(e.mean()) - 1.0) < 0.01 and abs(float(e.var()) - 1.0) < 0.03
    assert abs(float((e > 1.0).float().mean()) - math.exp(-1.0)) < 0.005
    # rows, offsets and seeds address different streams; the same address repeats
    assert not torch.equal(e[0], e[1])
    assert torch.equal(e, oracle.exponential_noise_oracle(7, 3, 4, 50001))
    assert not torch.equal(e, oracle.exponential_noise_oracle(7, 4, 4, 50001))
    assert not torch.equal(e, oracle.exponential_noise_oracle(8, 3, 4, 50001))
    # a shorter vocab is a prefix of the same stream
    assert torch.equal(oracle.exponential_noise_oracle(7, 3, 4, 10)[:, :10], e[:, :10])


def test_sampler_oracle_draws_from_the_tempered_softmax():
    g = torch.Generator().manual_seed(4)
    logits = torch.tensor([[2.0, 0.5, -1.0, 1.0, 0.0]]).repeat(40000, 1)
    temps = torch.full((40000,), 0.7)
    noise = torch.empty(40000, 5).exponential_(1.0, generator=g)
    ids = oracle.sampler_oracle(logits, temps, noise)
    freq = torch.bincount(ids, minlength=5).float() / 40000
    want = torch.softmax(logits[0] / 0.7, dim=-1)
    assert float((freq - want).abs().max()) < 0.01
    # the clamp: a zero draw does not divide by zero, it wins
    z = torch.ones(1, 5); z[0, 2] = 0.0
    assert int(oracle.sampler_oracle(logits[:1], temps[:1], z)) == 2


def test_silu_and_add_norm_oracles():
    g = torch.Generator().manual_seed(21)
    x = torch.randn(5, 32, generator=g) * 3
    got = oracle.silu_and_mul_oracle(x)
    assert torch.allclose(got, F.silu(x[:, :16]) * x[:, 16:], atol=1e-6)        # library routine
    a = x[:, :16]
    silu = lambda t: oracle.silu_and_mul_oracle(torch.cat([t, torch.ones_like(t)], dim=-1))
    assert torch.allclose(silu(a) - silu(-a), a, atol=1e-6)                     # x s(x) - (-x) s(-x) = x
    assert float(silu(torch.zeros(1, 4)).abs().max()) == 0.0
    assert torch.allclose(silu(torch.full((1, 4), 30.0)), torch.full((1, 4), 30.0))
    # bf16: the intermediate silu is rounded before the product
    xb = x.to(torch.bfloat16)
    two_step = (F.silu(xb[:, :16].float()).to(torch.bfloat16).float() * xb[:, 16:].float()).to(torch.bfloat16)
    assert torch.equal(oracle.silu_and_mul_oracle(xb), two_step)
    # residual form = norm of the rounded sum, returned with the sum
    r = torch.randn(5, 32, generator=g).to(torch.bfloat16)
    gamma = torch.rand(32, generator=g) + 0.5
    y, s = oracle.add_rms_norm_oracle(xb, gamma, 1e-6, r)
    assert torch.equal(s, xb + r) and torch.equal(y, oracle.rms_norm_oracle(xb + r, gamma, 1e-6))
    assert torch.equal(oracle.add_rms_norm_oracle(xb, gamma, 1e-6), oracle.rms_norm_oracle(xb, gamma, 1e-6))
