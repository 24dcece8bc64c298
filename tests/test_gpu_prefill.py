"""Causal varlen prefill attention on the GPU, through the C ABI, against the fp32 oracle."""
import pytest
import torch

import oracle
from nanovllm_amd import varlen_prefill_attention, store_kvcache
from nanovllm_amd import synthetic
from helpers import assert_attn_close, bits

pytestmark = pytest.mark.gpu


def _paged(case, dev):
    """scatter the new keys, then attend through the block table -- what Attention.forward does"""
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.k.to(dev), case.v.to(dev), kc, vc, case.slot_mapping.to(dev))
    out = varlen_prefill_attention(case.q.to(dev), kc, vc, case.cu_seqlens_q.to(dev), case.cu_seqlens_k.to(dev),
                                   case.max_seqlen_q, case.max_seqlen_k, case.scale,
                                   block_table=case.block_tables.to(dev))
    torch.cuda.synchronize()
    ek, ev = case.k_cache.clone(), case.v_cache.clone()
    oracle.store_kvcache(case.k, case.v, ek, ev, case.slot_mapping)
    want = oracle.varlen_prefill_attention(case.q, None, None, case.cu_seqlens_q, case.cu_seqlens_k, case.scale,
                                           ek, ev, case.block_tables, "fp32")
    return out, want


def _packed(case, dev, strided_v=False):
    k, v = case.k.to(dev), case.v.to(dev)
    if strided_v:
        n, hkv, dh = case.v.shape
        wide = torch.zeros(n, 4 * hkv * dh, dtype=torch.bfloat16, device=dev)
        wide[:, 3 * hkv * dh:] = v.reshape(n, -1)
        v = wide[:, 3 * hkv * dh:].view(n, hkv, dh)
    out = varlen_prefill_attention(case.q.to(dev), k, v, case.cu_seqlens_q.to(dev), case.cu_seqlens_k.to(dev),
                                   case.max_seqlen_q, case.max_seqlen_k, case.scale)
    torch.cuda.synchronize()
    want = oracle.varlen_prefill_attention(case.q, case.k, case.v, case.cu_seqlens_q, case.cu_seqlens_k,
                                           case.scale, precision="fp32")
    return out, want


def test_prefill_config3_prefix_cache(dev):
    """16 sequences, Lq U[100,1024], half with 1-3 cached 256-token prefix blocks."""
    case = synthetic.prefill_case(seed=0)
    assert case.block_tables is not None and sum(1 for p in case.prefix_lens if p) == 8
    out, want = _paged(case, dev)
    assert out.shape == case.q.shape
    assert_attn_close(out, want, "config 3")


@pytest.mark.parametrize("block_size", [512, 1024])
def test_prefill_larger_kv_blocks(dev, block_size):
    """KV blocks of 256 * 2^k tokens (nanovllm/config.py:22 allows multiples of 256): prefix blocks and the
    new tokens' slots follow the larger block."""
    case = synthetic.prefill_case(seed=block_size, batch=6, num_blocks=40, q_lo=50, q_hi=900, max_prefix_blocks=2,
                                  block_size=block_size)
    assert case.k_cache.shape[1] == block_size and any(case.prefix_lens)
    out, want = _paged(case, dev)
    assert_attn_close(out, want, f"block size {block_size}")


@pytest.mark.parametrize("strided_v", [False, True])
def test_prefill_no_prefix_packed(dev, strided_v):
    case = synthetic.prefill_case(seed=1, batch=6, prefix_fraction=0.0, q_lo=1, q_hi=700)
    assert case.block_tables is None
    out, want = _packed(case, dev, strided_v)
    assert_attn_close(out, want, "packed")


@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 8), (4, 1)])
def test_prefill_gqa_groups(dev, hq, hkv):
    case = synthetic.prefill_case(seed=hq, batch=4, num_heads=hq, num_kv_heads=hkv, q_lo=5, q_hi=400, num_blocks=24)
    out, want = _paged(case, dev)
    assert_attn_close(out, want, f"gqa {hq}/{hkv}")


def test_prefill_ragged_lengths_and_tile_edges(dev):
    q_lens = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300]
    prefix = [0, 1, 0, 2, 0, 0, 1, 0, 3, 0, 1, 0, 0, 2, 1]
    case = synthetic.prefill_case(seed=2, q_lens=q_lens, prefix_blocks=prefix, num_blocks=48)
    out, want = _paged(case, dev)
    assert_attn_close(out, want, "ragged paged")
    case2 = synthetic.prefill_case(seed=3, q_lens=q_lens, prefix_blocks=[0] * len(q_lens), num_blocks=48)
    out2, want2 = _packed(case2, dev)
    assert_attn_close(out2, want2, "ragged packed")
    # first token of every sequence sees one key only: output is exactly that V row
    for s in range(len(q_lens)):
        a = int(case2.cu_seqlens_q[s])
        assert torch.equal(bits(out2[a, 0]), bits(case2.v[a, 0]))
        assert torch.equal(bits(out2[a, 15]), bits(case2.v[a, 7]))


def test_prefill_lq1_with_prefix_equals_decode_semantics(dev):
    case = synthetic.prefill_case(seed=4, q_lens=[1, 1, 1], prefix_blocks=[1, 3, 2], num_blocks=16)
    out, want = _paged(case, dev)
    assert_attn_close(out, want, "lq=1")


def test_prefill_empty_query_span_is_a_noop(dev):
    """A prompt fully covered by cached blocks has seqlen_q == 0 (two equal cu_seqlens_q)."""
    case = synthetic.prefill_case(seed=5, q_lens=[40, 70], prefix_blocks=[1, 0], num_blocks=16)
    cu_q = torch.tensor([0, 40, 40, 110], dtype=torch.int32)
    cu_k = torch.tensor([0, 296, 296 + 512, 296 + 512 + 70], dtype=torch.int32)
    tables = torch.full((3, 2), -1, dtype=torch.int32)
    tables[0, :2] = case.block_tables[0, :2]
    tables[1, :2] = torch.tensor([14, 15], dtype=torch.int32)         # fully cached sequence
    tables[2, :1] = case.block_tables[1, :1]
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.k.to(dev), case.v.to(dev), kc, vc, case.slot_mapping.to(dev))
    out = varlen_prefill_attention(case.q.to(dev), kc, vc, cu_q.to(dev), cu_k.to(dev), 70, 512, case.scale,
                                   block_table=tables.to(dev))
    torch.cuda.synchronize()
    ek, ev = case.k_cache.clone(), case.v_cache.clone()
    oracle.store_kvcache(case.k, case.v, ek, ev, case.slot_mapping)
    want = oracle.varlen_prefill_attention(case.q, None, None, cu_q, cu_k, case.scale, ek, ev, tables, "fp32")
    assert_attn_close(out, want, "empty span")


def test_prefill_bad_table_entry_contributes_nothing(dev):
    """A block-table entry outside [0, num_blocks) must neither fault nor add anything: the keys of
    that block drop out.  Dropping whole prefix blocks leaves every remaining key visible to every
    query, so the expected result is the oracle's for the same sequences with a shorter prefix."""
    case = synthetic.prefill_case(seed=9, q_lens=[300, 150], prefix_blocks=[2, 1], num_blocks=32)
    t = case.block_tables
    bad = t.clone()
    bad[0, 1] = 9999                                    # second prefix block of sequence 0
    bad[1, 0] = -1                                      # the only prefix block of sequence 1
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.k.to(dev), case.v.to(dev), kc, vc, case.slot_mapping.to(dev))
    out = varlen_prefill_attention(case.q.to(dev), kc, vc, case.cu_seqlens_q.to(dev), case.cu_seqlens_k.to(dev),
                                   case.max_seqlen_q, case.max_seqlen_k, case.scale, block_table=bad.to(dev))
    torch.cuda.synchronize()
    ek, ev = case.k_cache.clone(), case.v_cache.clone()
    oracle.store_kvcache(case.k, case.v, ek, ev, case.slot_mapping)
    short = torch.full_like(t, -1)
    short[0, :3] = torch.stack([t[0, 0], t[0, 2], t[0, 3]])     # 256 prefix keys, then the 300 new ones
    short[1, :1] = t[1, 1]                                      # only the 150 new ones
    cu_k = torch.tensor([0, 256 + 300, 256 + 300 + 150], dtype=torch.int32)
    want = oracle.varlen_prefill_attention(case.q, None, None, case.cu_seqlens_q, cu_k, case.scale, ek, ev, short, "fp32")
    assert_attn_close(out, want, "bad table entries")


@pytest.mark.parametrize("bad_col", [0, 1])
def test_prefill_bad_table_entry_on_a_diagonal_tile_over_an_unwritten_cache(dev, bad_col):
    """A bad block id behind NEW tokens: its key tiles cross the causal diagonal (and one is the last
    tile of its query tile).  Every row of the caches that no token was written to -- block 0 above
    all, where a bad id's loads are pointed -- holds NaN bit patterns, as an engine's torch.empty
    cache may; the block's keys must drop out without a single NaN reaching the output."""
    g = torch.Generator().manual_seed(31 + bad_col)
    lq, hq, hkv, d = 300, 16, 8, 128
    q, k, v = (torch.randn(lq, h, d, generator=g).to(torch.bfloat16) for h in (hq, hkv, hkv))
    blocks = [3, 5]
    pos = torch.arange(lq)
    slots = (torch.tensor(blocks)[pos // 256] * 256 + pos % 256).to(torch.int32)
    kc = torch.full((8, 256, hkv, d), float("nan"), dtype=torch.bfloat16, device=dev)
    vc = torch.full_like(kc, float("nan"))
    store_kvcache(k.to(dev), v.to(dev), kc, vc, slots.to(dev))
    table = torch.tensor([blocks], dtype=torch.int32)
    table[0, bad_col] = 9999 if bad_col else -1
    cu = torch.tensor([0, lq], dtype=torch.int32)
    out = varlen_prefill_attention(q.to(dev), kc, vc, cu.to(dev), cu.to(dev), lq, lq, d ** -0.5, block_table=table.to(dev))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out.float()).all()), "NaN from an unwritten block reached the output"
    scale = d ** -0.5
    if bad_col == 1:
        # keys 256.. drop out: queries below 256 are untouched, the others see keys 0..255, all of them
        cu256 = torch.tensor([0, 256], dtype=torch.int32)
        low = oracle.varlen_prefill_attention(q[:256], k[:256], v[:256], cu256, cu256, scale, precision="fp32")
        n = lq - 256
        cu_q1 = torch.arange(n + 1, dtype=torch.int32)
        cu_k1 = (torch.arange(n + 1) * 256).to(torch.int32)
        high = oracle.varlen_prefill_attention(q[256:], k[:256].repeat(n, 1, 1), v[:256].repeat(n, 1, 1), cu_q1, cu_k1,
                                               scale, precision="fp32")
        want = torch.cat([low, high])
    else:
        # keys 0..255 drop out: queries below 256 see nothing (zero rows), the others the keys from 256 on, causally
        cu_t = torch.tensor([0, lq - 256], dtype=torch.int32)
        high = oracle.varlen_prefill_attention(q[256:], k[256:], v[256:], cu_t, cu_t, scale, precision="fp32")
        want = torch.cat([torch.zeros(256, hq, d), high])
    assert_attn_close(out, want, f"bad id in column {bad_col}")


def test_prefill_sequences_do_not_leak(dev):
    case = synthetic.prefill_case(seed=6, batch=3, prefix_fraction=0.0, q_lo=50, q_hi=200)
    out, _ = _packed(case, dev)
    k2 = case.k.clone()
    a, b = int(case.cu_seqlens_q[1]), int(case.cu_seqlens_q[2])
    k2[a:b] = 2.0
    case2 = synthetic.PrefillCase(case.q, k2, case.v, case.k_cache, case.v_cache, case.cu_seqlens_q,
                                  case.cu_seqlens_k, case.max_seqlen_q, case.max_seqlen_k, case.slot_mapping,
                                  None, case.scale)
    out2, _ = _packed(case2, dev)
    assert torch.equal(bits(out[:a]), bits(out2[:a])) and torch.equal(bits(out[b:]), bits(out2[b:]))
    assert not torch.equal(bits(out[a:b]), bits(out2[a:b]))


def test_prefill_warmup_shape_4x4096(dev):
    """The runner's warm-up batch (4 sequences of max_model_len = 4096 tokens, packed, no cache):
    64 key tiles per row, far more than config 3 has.  One sequence is checked against the fp32
    oracle in full; every sequence launched alone, and the same four packed in another order, give
    the same bits as inside the batch (a row's arithmetic does not depend on what else is in the
    launch -- this is the check that catches a missed hardware wait state, which moves a result by
    far less than the tolerance)."""
    g = torch.Generator().manual_seed(21)
    n, L = 4, 4096
    q = (torch.randn((n * L, 16, 128), generator=g)).to(torch.bfloat16)
    k = (torch.randn((n * L, 8, 128), generator=g)).to(torch.bfloat16)
    v = (torch.randn((n * L, 8, 128), generator=g)).to(torch.bfloat16)
    cu = torch.arange(0, (n + 1) * L, L, dtype=torch.int32)
    scale = 128 ** -0.5
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = varlen_prefill_attention(qd, kd, vd, cu.to(dev), cu.to(dev), L, L, scale)
    torch.cuda.synchronize()
    one = torch.tensor([0, L], dtype=torch.int32)
    s = 2                                                        # the sequence given to the oracle
    want = oracle.varlen_prefill_attention(q[s * L:(s + 1) * L], k[s * L:(s + 1) * L], v[s * L:(s + 1) * L], one, one,
                                           scale, precision="fp32")
    assert_attn_close(out[s * L:(s + 1) * L], want, "4096-token sequence")
    order = [2, 0, 3, 1]
    pick = torch.cat([torch.arange(i * L, (i + 1) * L) for i in order]).to(dev)
    again = varlen_prefill_attention(qd[pick], kd[pick], vd[pick], cu.to(dev), cu.to(dev), L, L, scale)
    for j, i in enumerate(order):
        assert torch.equal(bits(again[j * L:(j + 1) * L]), bits(out[i * L:(i + 1) * L]))
    for i in range(n):
        alone = varlen_prefill_attention(qd[i * L:(i + 1) * L], kd[i * L:(i + 1) * L], vd[i * L:(i + 1) * L],
                                         one.to(dev), one.to(dev), L, L, scale)
        assert torch.equal(bits(alone), bits(out[i * L:(i + 1) * L]))


@pytest.mark.parametrize("hq,hkv,q_lens", [(4, 1, [4096, 300]), (16, 8, [2000, 100, 70, 1]), (2, 2, [1500])])
def test_prefill_one_sequence_dominates(dev, hq, hkv, q_lens):
    """Ragged batches in which one long sequence sits beside very short ones (query tiles of 2 to 64
    key tiles in one launch), packed and through the block table, few heads and many."""
    case = synthetic.prefill_case(seed=hq * 7, q_lens=q_lens, prefix_blocks=[0] * len(q_lens), num_heads=hq,
                                  num_kv_heads=hkv, num_blocks=32)
    out, want = _packed(case, dev)
    assert_attn_close(out, want, "dominant sequence, packed")
    prefix = [2] + [0] * (len(q_lens) - 1)
    case = synthetic.prefill_case(seed=hq * 7 + 1, q_lens=q_lens, prefix_blocks=prefix, num_heads=hq, num_kv_heads=hkv,
                                  num_blocks=40)
    out, want = _paged(case, dev)
    assert_attn_close(out, want, "dominant sequence, paged")


@pytest.mark.parametrize("boost_from,factor", [(32, 40.0), (200, 60.0), (0, 50.0)])
def test_prefill_scores_far_beyond_the_first_keys(dev, boost_from, factor):
    """The kernel takes its exponent reference from the first 32 keys of a row and repeats a query
    tile with exact row maxima when a row sum shows that this was not enough.  Keys from
    `boost_from` on are scaled so that their scores exceed the first keys' by many hundreds (raw
    score standard deviation ~ 11 * factor), which overflows every p computed against the cheap
    reference; with boost_from = 0 the large scores are in the first keys instead and everything
    after them underflows.  Packed and through the block table; rows see between 1 and ~900 keys."""
    q_lens, prefix = [300, 129, 64, 500], [1, 0, 2, 0]
    case = synthetic.prefill_case(seed=31, q_lens=q_lens, prefix_blocks=[0] * 4, num_blocks=40)
    k = case.k.clone()
    for s in range(len(q_lens)):
        a, b = int(case.cu_seqlens_q[s]), int(case.cu_seqlens_q[s + 1])
        if boost_from == 0:
            k[a:min(a + 20, b)] = (k[a:min(a + 20, b)].float() * factor).to(torch.bfloat16)
        elif a + boost_from < b:
            k[a + boost_from:b] = (k[a + boost_from:b].float() * factor).to(torch.bfloat16)
    packed = synthetic.PrefillCase(case.q, k, case.v, case.k_cache, case.v_cache, case.cu_seqlens_q, case.cu_seqlens_k,
                                   case.max_seqlen_q, case.max_seqlen_k, case.slot_mapping, None, case.scale)
    out, want = _packed(packed, dev)
    assert_attn_close(out, want, f"boosted keys from {boost_from}, packed")
    paged = synthetic.prefill_case(seed=32, q_lens=q_lens, prefix_blocks=prefix, num_blocks=40)
    k2 = paged.k.clone()
    for s in range(len(q_lens)):
        a, b = int(paged.cu_seqlens_q[s]), int(paged.cu_seqlens_q[s + 1])
        lo = a if boost_from == 0 else min(a + boost_from, b)
        hi = min(a + 20, b) if boost_from == 0 else b
        k2[lo:hi] = (k2[lo:hi].float() * factor).to(torch.bfloat16)
    paged = synthetic.PrefillCase(paged.q, k2, paged.v, paged.k_cache, paged.v_cache, paged.cu_seqlens_q,
                                  paged.cu_seqlens_k, paged.max_seqlen_q, paged.max_seqlen_k, paged.slot_mapping,
                                  paged.block_tables, paged.scale)
    out, want = _paged(paged, dev)
    assert_attn_close(out, want, f"boosted keys from {boost_from}, paged")


def test_prefill_rows_without_any_key_are_zero(dev):
    """More queries than keys (cu_seqlens_k shorter than cu_seqlens_q): with the mask aligned to the end
    of the keys the first Lq - Lk queries see nothing and come out as zeros, as the oracle's do."""
    g = torch.Generator().manual_seed(41)
    lq, lk = 200, 70
    q = torch.randn((lq, 4, 128), generator=g).to(torch.bfloat16)
    k = torch.randn((lk, 2, 128), generator=g).to(torch.bfloat16)
    v = torch.randn((lk, 2, 128), generator=g).to(torch.bfloat16)
    cu_q, cu_k = torch.tensor([0, lq], dtype=torch.int32), torch.tensor([0, lk], dtype=torch.int32)
    out = varlen_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu_q.to(dev), cu_k.to(dev), lq, lk, 128 ** -0.5)
    torch.cuda.synchronize()
    want = oracle.varlen_prefill_attention(q, k, v, cu_q, cu_k, 128 ** -0.5, precision="fp32")
    assert float(want[:lq - lk].abs().max()) == 0.0
    assert float(out[:lq - lk].float().abs().max()) == 0.0
    assert_attn_close(out, want, "more queries than keys")
