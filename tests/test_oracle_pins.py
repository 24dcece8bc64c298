"""Pins for the CPU oracle (oracle/hotpath.py).

The reference ships no golden vectors for this path, so each oracle function is pinned
against things it does not share code with: float64 pure-Python loops written from the
textbook definitions, torch library routines on special cases, and invariants chosen so
that a dropped term, a wrong head mapping, a mis-aligned mask or a transposed index fails.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle


def _rand_bf16(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(torch.bfloat16)


# ------------------------------------------------------------------ brute-force definitions
def brute_attention(q, keys, values, scale, q_offset):
    """q [Lq][Hq][D], keys/values [Lk][Hkv][D] python lists of floats -> [Lq][Hq][D]."""
    lq, hq, d = len(q), len(q[0]), len(q[0][0])
    lk, hkv = len(keys), len(keys[0]) if keys else 1
    group = hq // hkv
    out = [[[0.0] * d for _ in range(hq)] for _ in range(lq)]
    for i in range(lq):
        for h in range(hq):
            g = h // group
            vis = [j for j in range(lk) if j <= i + q_offset]
            if not vis:
                continue
            s = [scale * sum(q[i][h][x] * keys[j][g][x] for x in range(d)) for j in vis]
            m = max(s)
            w = [math.exp(v - m) for v in s]
            z = sum(w)
            for x in range(d):
                out[i][h][x] = sum(w[n] * values[j][g][x] for n, j in enumerate(vis)) / z
    return out


def brute_gather(cache, table_row, n):
    page = cache.shape[1]
    return [cache[int(table_row[p // page]), p % page].float().tolist() for p in range(n)]


# ------------------------------------------------------------------ scatter
def test_scatter_matches_python_loop():
    g = torch.Generator().manual_seed(1)
    n, hkv, dh, slots = 37, 2, 8, 64
    key, value = _rand_bf16(n, hkv, dh, seed=2), _rand_bf16(n, hkv, dh, seed=3)
    sm = torch.randperm(slots, generator=g)[:n].to(torch.int32)
    sm[[3, 11, 36]] = -1
    kc = torch.zeros(slots // 4, 4, hkv, dh, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    oracle.store_kvcache(key, value, kc, vc, sm)
    exp_k = torch.zeros(slots, hkv * dh, dtype=torch.bfloat16)
    exp_v = torch.zeros_like(exp_k)
    for i in range(n):
        s = int(sm[i])
        if s == -1:
            continue
        for x in range(hkv * dh):
            exp_k[s, x] = key.reshape(n, -1)[i, x]
            exp_v[s, x] = value.reshape(n, -1)[i, x]
    assert torch.equal(kc.view(slots, -1).view(torch.int16), exp_k.view(torch.int16))
    assert torch.equal(vc.view(slots, -1).view(torch.int16), exp_v.view(torch.int16))


def test_scatter_invariants():
    n, hkv, dh, slots = 50, 2, 8, 128
    key, value = _rand_bf16(n, hkv, dh, seed=4), _rand_bf16(n, hkv, dh, seed=5)
    g = torch.Generator().manual_seed(6)
    sm = torch.randperm(slots, generator=g)[:n].to(torch.int32)
    kc = torch.zeros(slots, hkv, dh, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    # all -1: nothing changes
    oracle.store_kvcache(key, value, kc, vc, torch.full((n,), -1, dtype=torch.int32))
    assert not kc.any() and not vc.any()
    oracle.store_kvcache(key, value, kc, vc, sm)
    # untouched slots stay zero, touched slots hold the row; K never lands in V
    touched = torch.zeros(slots, dtype=torch.bool)
    touched[sm.long()] = True
    assert not kc[~touched].any() and not vc[~touched].any()
    assert torch.equal(kc[sm.long()], key) and torch.equal(vc[sm.long()], value)
    # token order does not matter when slots are unique
    perm = torch.randperm(n, generator=g)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    oracle.store_kvcache(key[perm], value[perm], kc2, vc2, sm[perm])
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    # strided value view (as in the fused qkv buffer) gives the same cache
    wide = torch.zeros(n, 3 * hkv * dh, dtype=torch.bfloat16)
    wide[:, hkv * dh: 2 * hkv * dh] = value.reshape(n, -1)
    v_view = wide[:, hkv * dh: 2 * hkv * dh].view(n, hkv, dh)
    kc3, vc3 = torch.zeros_like(kc), torch.zeros_like(vc)
    oracle.store_kvcache(key, v_view, kc3, vc3, sm)
    assert torch.equal(vc, vc3)


# ------------------------------------------------------------------ block-table indexing
def test_gather_pages_position_formula():
    nb, page, hkv, dh = 7, 4, 2, 3
    cache = torch.arange(nb * page * hkv * dh, dtype=torch.float32).view(nb, page, hkv, dh)
    table = torch.tensor([5, 2, 6, -1, -1], dtype=torch.int32)
    n = 10   # needs ceil(10/4)=3 entries; the -1 padding must never be touched
    got = oracle.gather_pages(cache, table, n)
    assert got.shape == (n, hkv, dh)
    for p in range(n):
        assert torch.equal(got[p], cache[int(table[p // page]), p % page])


# ------------------------------------------------------------------ decode attention
@pytest.mark.parametrize("hq,hkv", [(4, 2), (4, 1), (2, 2)])
def test_decode_matches_float64_loops(hq, hkv):
    b, dh, page, nb = 3, 8, 4, 12
    q = _rand_bf16(b, hq, dh, seed=10)
    kc, vc = _rand_bf16(nb, page, hkv, dh, seed=11), _rand_bf16(nb, page, hkv, dh, seed=12)
    ctx = torch.tensor([1, 6, 11], dtype=torch.int32)
    tables = torch.tensor([[7, -1, -1], [3, 9, -1], [0, 11, 5]], dtype=torch.int32)
    scale = 0.37
    got = oracle.paged_decode_attention(q, kc, vc, ctx, tables, scale, "fp32")
    assert got.shape == (b, 1, hq, dh)
    for s in range(b):
        n = int(ctx[s])
        want = brute_attention([q[s].float().tolist()], brute_gather(kc, tables[s], n),
                               brute_gather(vc, tables[s], n), scale, n - 1)
        assert torch.allclose(got[s, 0].double(), torch.tensor(want[0], dtype=torch.float64), atol=2e-6)


def test_decode_special_cases_and_invariants():
    b, hq, hkv, dh, page, nb = 4, 4, 2, 16, 8, 16
    q = _rand_bf16(b, hq, dh, seed=20)
    kc, vc = _rand_bf16(nb, page, hkv, dh, seed=21), _rand_bf16(nb, page, hkv, dh, seed=22)
    ctx = torch.tensor([0, 1, 8, 19], dtype=torch.int32)
    tables = torch.tensor([[-1, -1, -1], [4, -1, -1], [9, -1, -1], [2, 13, 6]], dtype=torch.int32)
    out = oracle.paged_decode_attention(q, kc, vc, ctx, tables, 0.25, "fp32")
    # context_len 0 -> zeros
    assert not out[0].any()
    # one key -> output is that V row, heads 2g and 2g+1 read kv head g
    assert torch.equal(out[1, 0, 0], vc[4, 0, 0].float()) and torch.equal(out[1, 0, 1], vc[4, 0, 0].float())
    assert torch.equal(out[1, 0, 2], vc[4, 0, 1].float()) and torch.equal(out[1, 0, 3], vc[4, 0, 1].float())
    # V == 1 -> out == 1
    ones = oracle.paged_decode_attention(q, kc, torch.ones_like(vc), ctx, tables, 0.25, "fp32")
    assert torch.allclose(ones[1:], torch.ones_like(ones[1:]), atol=1e-6)
    # library special case: dense SDPA on the gathered keys (library does the softmax)
    n = 19
    k = oracle.gather_pages(kc, tables[3], n).float()
    v = oracle.gather_pages(vc, tables[3], n).float()
    want = F.scaled_dot_product_attention(
        q[3].float().view(1, hq, 1, dh), k.permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0),
        v.permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0), scale=0.25)
    assert torch.allclose(out[3, 0], want[0, :, 0], atol=1e-5)
    # physical block permutation invariance
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(23))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb)
    kc2, vc2 = kc[perm], vc[perm]          # block i of the new pool = old block perm[i]
    t2 = torch.where(tables >= 0, inv[tables.clamp_min(0).long()].to(torch.int32), tables)
    out2 = oracle.paged_decode_attention(q, kc2, vc2, ctx, t2, 0.25, "fp32")
    assert torch.equal(out, out2)
    # keys beyond context_len are ignored
    kc3, vc3 = kc.clone(), vc.clone()
    kc3[6, 3:], vc3[6, 3:] = 1e4, 1e4      # block 6 holds positions 16..23 of seq 3; ctx = 19
    out3 = oracle.paged_decode_attention(q, kc3, vc3, ctx, tables, 0.25, "fp32")
    assert torch.equal(out, out3)
    # bf16 SDPA mode (the timed CPU baseline) agrees with fp32 to bf16 accuracy
    sd = oracle.paged_decode_attention(q, kc, vc, ctx, tables, 0.25, "sdpa")
    assert sd.dtype == torch.bfloat16 and (sd.float() - out).abs().max() < 3e-2


# ------------------------------------------------------------------ prefill attention
def test_prefill_matches_float64_loops_with_prefix():
    hq, hkv, dh, page, nb = 4, 2, 8, 4, 16
    q_lens, prefix = [3, 5, 2], [4, 0, 8]
    k_lens = [a + p for a, p in zip(q_lens, prefix)]
    tq = sum(q_lens)
    q = _rand_bf16(tq, hq, dh, seed=30)
    kc, vc = _rand_bf16(nb, page, hkv, dh, seed=31), _rand_bf16(nb, page, hkv, dh, seed=32)
    tables = torch.tensor([[3, 8, -1], [5, 1, -1], [10, 2, 7]], dtype=torch.int32)
    cu_q = torch.tensor([0, 3, 8, 10], dtype=torch.int32)
    cu_k = torch.tensor([0, 7, 12, 22], dtype=torch.int32)
    got = oracle.varlen_prefill_attention(q, None, None, cu_q, cu_k, 0.3, kc, vc, tables, "fp32")
    for s in range(3):
        want = brute_attention(q[int(cu_q[s]):int(cu_q[s + 1])].float().tolist(),
                               brute_gather(kc, tables[s], k_lens[s]), brute_gather(vc, tables[s], k_lens[s]),
                               0.3, k_lens[s] - q_lens[s])
        assert torch.allclose(got[int(cu_q[s]):int(cu_q[s + 1])].double(),
                              torch.tensor(want, dtype=torch.float64), atol=2e-6)


def test_prefill_special_cases():
    hq, hkv, dh = 4, 2, 16
    q_lens = [5, 1, 9]
    tq = sum(q_lens)
    q, k, v = _rand_bf16(tq, hq, dh, seed=40), _rand_bf16(tq, hkv, dh, seed=41), _rand_bf16(tq, hkv, dh, seed=42)
    cu = torch.tensor([0, 5, 6, 15], dtype=torch.int32)
    out = oracle.varlen_prefill_attention(q, k, v, cu, cu, 0.25, precision="fp32")
    # no prefix: equals the library's top-left causal attention per sequence
    for s in range(3):
        a, b = int(cu[s]), int(cu[s + 1])
        want = F.scaled_dot_product_attention(
            q[a:b].float().permute(1, 0, 2).unsqueeze(0),
            k[a:b].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0),
            v[a:b].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0), is_causal=True, scale=0.25)
        assert torch.allclose(out[a:b], want[0].permute(1, 0, 2), atol=1e-5)
    # first query of a sequence sees exactly one key: output = that V row (no leak across cu_seqlens)
    assert torch.equal(out[5, 0], v[5, 0].float()) and torch.equal(out[6, 3], v[6, 1].float())
    # sequences are independent: changing sequence 0's keys leaves the others alone
    k2 = k.clone()
    k2[:5] = 3.0
    out2 = oracle.varlen_prefill_attention(q, k2, v, cu, cu, 0.25, precision="fp32")
    assert torch.equal(out[5:], out2[5:]) and not torch.equal(out[:5], out2[:5])
    # an empty query span is a no-op
    cu_q = torch.tensor([0, 5, 5, 6], dtype=torch.int32)
    cu_k = torch.tensor([0, 5, 9, 10], dtype=torch.int32)
    out3 = oracle.varlen_prefill_attention(q[:6], k[:10], v[:10], cu_q, cu_k, 0.25, precision="fp32")
    assert out3.shape[0] == 6


def test_prefill_lq1_with_prefix_equals_decode_and_paged_equals_packed():
    hq, hkv, dh, page, nb = 4, 2, 16, 8, 8
    kc, vc = _rand_bf16(nb, page, hkv, dh, seed=50), _rand_bf16(nb, page, hkv, dh, seed=51)
    tables = torch.tensor([[6, 1, 3], [2, 7, -1]], dtype=torch.int32)
    lk = [19, 13]
    q = _rand_bf16(2, hq, dh, seed=52)
    cu_q = torch.tensor([0, 1, 2], dtype=torch.int32)
    cu_k = torch.tensor([0, 19, 32], dtype=torch.int32)
    pre = oracle.varlen_prefill_attention(q, None, None, cu_q, cu_k, 0.25, kc, vc, tables, "fp32")
    dec = oracle.paged_decode_attention(q, kc, vc, torch.tensor(lk, dtype=torch.int32), tables, 0.25, "fp32")
    assert torch.equal(pre, dec[:, 0])
    # bottom-right alignment: several queries with a prefix; paged and packed keys agree
    q_lens, cu_q2 = [4, 5], torch.tensor([0, 4, 9], dtype=torch.int32)
    q2 = _rand_bf16(9, hq, dh, seed=53)
    paged = oracle.varlen_prefill_attention(q2, None, None, cu_q2, cu_k, 0.25, kc, vc, tables, "fp32")
    kd = torch.cat([oracle.gather_pages(kc, tables[s], lk[s]) for s in range(2)])
    vd = torch.cat([oracle.gather_pages(vc, tables[s], lk[s]) for s in range(2)])
    packed = oracle.varlen_prefill_attention(q2, kd, vd, cu_q2, cu_k, 0.25, precision="fp32")
    assert torch.equal(paged, packed)
    # the LAST query sees every key: equals non-causal attention over all Lk keys
    full = F.scaled_dot_product_attention(
        q2[3].float().view(1, hq, 1, dh), kd[:19].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0),
        vd[:19].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0), scale=0.25)
    assert torch.allclose(packed[3], full[0, :, 0], atol=1e-5)
    # the FIRST query of sequence 0 sees exactly Lk - Lq + 1 = 16 keys
    first = F.scaled_dot_product_attention(
        q2[0].float().view(1, hq, 1, dh), kd[:16].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0),
        vd[:16].float().permute(1, 0, 2).repeat_interleave(2, 0).unsqueeze(0), scale=0.25)
    assert torch.allclose(packed[0], first[0, :, 0], atol=1e-5)


# ------------------------------------------------------------------ sampler
def test_sampler_matches_float64_definition():
    g = torch.Generator().manual_seed(60)
    b, v = 16, 97
    logits = (torch.randn(b, v, generator=g) * 3).to(torch.bfloat16)
    temps = torch.rand(b, generator=g) + 0.3
    noise = torch.empty(b, v).exponential_(1.0, generator=g)
    got = oracle.sample(logits, temps, noise)
    assert got.dtype == torch.int64 and got.shape == (b,)
    for r in range(b):
        x = [float(logits[r, i]) / float(temps[r]) for i in range(v)]
        m = max(x)
        w = [math.exp(a - m) for a in x]
        z = sum(w)
        score = [w[i] / z / max(float(noise[r, i]), 1e-10) for i in range(v)]
        best = max(range(v), key=lambda i: score[i])
        top2 = sorted(score, reverse=True)[:2]
        if (top2[0] - top2[1]) > 1e-5 * top2[0]:      # skip fp32 near-ties
            assert int(got[r]) == best


def test_sampler_invariants():
    g = torch.Generator().manual_seed(61)
    b, v = 8, 300
    logits = (torch.randn(b, v, generator=g) * 2).to(torch.bfloat16)
    temps = torch.full((b,), 0.6)
    ones = torch.ones(b, v)
    # E == 1 -> plain argmax of the logits (ties: first index)
    assert torch.equal(oracle.sample(logits, temps, ones), logits.float().argmax(-1))
    # clamp: a zero noise entry wins unless its probability underflows
    noise = torch.ones(b, v)
    noise[:, 17] = 0.0
    assert torch.equal(oracle.sample(logits, temps, noise), torch.full((b,), 17))
    # temperature 0 rows are greedy regardless of noise
    t0 = temps.clone()
    t0[::2] = 0.0
    rnd = torch.empty(b, v).exponential_(1.0, generator=g)
    tok = oracle.sample(logits, t0, rnd)
    assert torch.equal(tok[::2], logits.float().argmax(-1)[::2])
    # inputs are not modified (the reference clamps its private noise tensor in place)
    noise_before = noise.clone()
    oracle.sample(logits, temps, noise)
    assert torch.equal(noise, noise_before)
    # equivalent Gumbel form argmax(x - log E) away from ties
    x = logits.float() / temps[:, None]
    alt = (x - rnd.clamp_min(1e-10).log()).argmax(-1)
    same = (oracle.sample(logits, temps, rnd) == alt).float().mean()
    assert same == 1.0


def test_sampler_is_a_categorical_draw():
    # chi-square of empirical token frequencies against softmax(logits / T)
    g = torch.Generator().manual_seed(62)
    v, n = 12, 40000
    logits = torch.tensor([[2.0, 1.0, 0.5, 0.0, -0.5, -1.0, 1.5, 0.25, -2.0, 0.75, -0.25, 1.25]]).to(torch.bfloat16)
    t = 0.8
    rows = logits.expand(n, v).contiguous()
    noise = torch.empty(n, v).exponential_(1.0, generator=g)
    tok = oracle.sample(rows, torch.full((n,), t), noise)
    freq = torch.bincount(tok, minlength=v).double()
    p = torch.softmax(logits.double()[0] / t, -1)
    chi2 = float(((freq - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 40.0     # 11 dof: P(chi2 > 40) ~ 4e-5


# ------------------------------------------------------------------ draws without a noise tensor
def test_philox_known_answers():
    """Known-answer vectors of Philox4x32-10 from the authors' Random123 distribution
    (kat_vectors: counter words, key words -> output words)."""
    assert oracle.philox4x32_10((0, 0, 0, 0), (0, 0)) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert oracle.philox4x32_10((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert oracle.philox4x32_10((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0)) == [
        0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    u = oracle.row_uniforms(seed=7, offset=3, batch=2000)
    assert float(u.min()) > 0 and float(u.max()) < 1
    assert abs(float(u.mean()) - 0.5) < 0.03 and not torch.equal(u, oracle.row_uniforms(7, 4, 2000))


def test_inverse_cdf_draws_the_softmax():
    """Walking the running sums with an even grid of uniforms reproduces every probability to
    within one grid step: the draw is categorical in softmax(logits / T), like the race."""
    row = torch.tensor([[2.0, 1.0, 0.5, 0.0, -0.5, -1.0, 1.5, 0.25]]).to(torch.bfloat16)
    t = torch.tensor([0.7])
    bounds = oracle.inverse_cdf_bounds(row, t)[0]
    assert abs(float(bounds[-1]) - 1.0) < 1e-12 and bool((bounds[1:] >= bounds[:-1]).all())
    n = 100000
    u = (torch.arange(n, dtype=torch.float64) + 0.5) / n
    tok = torch.searchsorted(bounds, u, right=True).clamp_max(row.shape[1] - 1)
    freq = torch.bincount(tok, minlength=row.shape[1]).double() / n
    p = torch.softmax(row[0].double() / 0.7, -1)
    assert float((freq - p).abs().max()) <= 1.0 / n + 1e-12


def test_tree_draw_reduces_to_one_inverse_cdf_on_eight_columns():
    """With at most 8 columns only the last level of the tree has a choice, so the draw must be the
    plain inverse CDF of that level's uniform: word 2 of Philox counter (row, 0x10000, offset)."""
    g = torch.Generator().manual_seed(8)
    batch, seed, offset = 300, 0xABCDEF0123, 41
    logits = (torch.randn(batch, 8, generator=g) * 1.5).to(torch.bfloat16)
    logits[::7, 2] = float("-inf")
    temps = torch.linspace(0.4, 1.6, batch)
    tok, margin = oracle.tree_draw(logits, temps, seed, offset)
    bounds = oracle.inverse_cdf_bounds(logits, temps)
    u = torch.tensor([(oracle.philox4x32_10((b, 0x10000, offset, 0), (seed & 0xFFFFFFFF, seed >> 32))[2] + 0.5) * 2.0 ** -32
                      for b in range(batch)], dtype=torch.float64)
    want = torch.searchsorted(bounds, u.unsqueeze(1), right=True).squeeze(1)
    sure = margin > 1e-9
    assert int(sure.sum()) >= batch - 2 and torch.equal(tok[sure], want[sure])
    assert bool((logits[torch.arange(batch), tok] > float("-inf")).all())


def test_tree_draw_is_categorical_across_all_levels():
    """Heavy columns placed so that every level of the tree has to choose (different chunks, column
    groups, lanes, and columns of one lane in the same and in different 2048-column slices):
    empirical frequencies over many rows against softmax(logits / T), chi-square."""
    cols = [3, 5, 6, 11, 700, 2050, 2051, 4100, 8191, 8192, 9000, 16390, 19999]
    vocab, n, t = 20000, 12000, 0.9
    row = torch.full((vocab,), float("-inf"))
    vals = torch.tensor([1.0, 0.5, 2.0, 0.0, 1.5, -0.5, 0.25, 1.0, 0.75, 2.0, -1.0, 1.25, 0.5])
    row[cols] = vals
    logits = row.to(torch.bfloat16).expand(n, vocab)
    tok, _ = oracle.tree_draw(logits, torch.full((n,), t), seed=99, offset=5)
    p = torch.softmax(vals.double() / t, -1)
    index = {c: i for i, c in enumerate(cols)}
    assert all(int(x) in index for x in tok.tolist())            # never a column of zero weight
    freq = torch.bincount(torch.tensor([index[int(x)] for x in tok.tolist()]), minlength=len(cols)).double()
    chi2 = float(((freq - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 45.0, chi2                                      # 12 dof: P(chi2 > 45) ~ 1e-5
    # a different offset is a different draw; the same key reproduces it
    again, _ = oracle.tree_draw(logits[:50], torch.full((50,), t), seed=99, offset=5)
    other, _ = oracle.tree_draw(logits[:50], torch.full((50,), t), seed=99, offset=6)
    assert torch.equal(again, tok[:50]) and not torch.equal(other, tok[:50])
