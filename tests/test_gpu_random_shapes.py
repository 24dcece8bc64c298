"""Seeded sweeps over head geometries, batch sizes and length ranges: decode and prefill attention
through the C ABI against the fp32 oracle, plus bit-identical repeats (a row's arithmetic must not
depend on how often or in which company it is computed)."""
import random

import pytest
import torch

import oracle
from nanovllm_amd import paged_decode_attention, varlen_prefill_attention, store_kvcache, synthetic
from nanovllm_amd.context import DecodePlan
from helpers import assert_attn_close

pytestmark = pytest.mark.gpu


def _decode_cases(seed, n):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        hkv, g = rng.choice([1, 2, 4, 8]), rng.choice([1, 2, 4, 8])
        batch, hi = rng.choice([1, 2, 3, 7, 16, 33, 100]), rng.choice([40, 300, 1100, 3000])
        lo = rng.choice([0, 1, hi // 2])
        blocks = max(16, batch * ((hi + 255) // 256) + 4)
        if hkv * g > 32 or blocks * 256 * hkv * 128 * 4 > 1.0e9:
            continue
        out.append((len(out), batch, hkv * g, hkv, lo, hi, blocks))
    return out


def _prefill_cases(seed, n):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        hkv, g = rng.choice([1, 2, 8]), rng.choice([1, 2, 4])
        out.append((i, rng.choice([1, 2, 5, 9]), hkv * g, hkv, rng.choice([30, 200, 700, 1500]), rng.choice([0.0, 0.5, 1.0])))
    return out


@pytest.mark.parametrize("i,batch,hq,hkv,lo,hi,blocks", _decode_cases(11, 24))
def test_decode_random_shape(dev, i, batch, hq, hkv, lo, hi, blocks):
    case = synthetic.decode_case(seed=1000 + i, batch=batch, num_heads=hq, num_kv_heads=hkv, num_blocks=blocks,
                                 ctx_lo=lo, ctx_hi=hi)
    d = (case.q.to(dev), case.k_cache.to(dev), case.v_cache.to(dev), case.context_lens.to(dev), case.block_tables.to(dev))
    out = paged_decode_attention(*d, case.scale).clone()
    want = oracle.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.context_lens, case.block_tables,
                                         case.scale, "fp32")
    assert_attn_close(out, want, f"decode batch {batch} heads {hq}/{hkv} ctx [{lo},{hi}]")
    plan = DecodePlan()
    for _ in range(3):                                   # the work split is built once, then reused
        assert torch.equal(paged_decode_attention(*d, case.scale, plan=plan), out)


@pytest.mark.parametrize("i,batch,hq,hkv,q_hi,prefix_fraction", _prefill_cases(12, 20))
def test_prefill_random_shape(dev, i, batch, hq, hkv, q_hi, prefix_fraction):
    case = synthetic.prefill_case(seed=2000 + i, batch=batch, num_heads=hq, num_kv_heads=hkv, num_blocks=batch * 10 + 8,
                                  q_lo=1, q_hi=q_hi, prefix_fraction=prefix_fraction, max_prefix_blocks=3)
    kc, vc = case.k_cache.to(dev), case.v_cache.to(dev)
    store_kvcache(case.k.to(dev), case.v.to(dev), kc, vc, case.slot_mapping.to(dev))
    cu_q, cu_k = case.cu_seqlens_q.to(dev), case.cu_seqlens_k.to(dev)
    if case.block_tables is not None:
        ek, ev = case.k_cache.clone(), case.v_cache.clone()
        oracle.store_kvcache(case.k, case.v, ek, ev, case.slot_mapping)
        run = lambda: varlen_prefill_attention(case.q.to(dev), kc, vc, cu_q, cu_k, case.max_seqlen_q, case.max_seqlen_k,
                                               case.scale, block_table=case.block_tables.to(dev))
        want = oracle.varlen_prefill_attention(case.q, None, None, case.cu_seqlens_q, case.cu_seqlens_k, case.scale,
                                               ek, ev, case.block_tables, "fp32")
    else:
        run = lambda: varlen_prefill_attention(case.q.to(dev), case.k.to(dev), case.v.to(dev), cu_q, cu_k,
                                               case.max_seqlen_q, case.max_seqlen_k, case.scale)
        want = oracle.varlen_prefill_attention(case.q, case.k, case.v, case.cu_seqlens_q, case.cu_seqlens_k, case.scale,
                                               precision="fp32")
    out = run()
    torch.cuda.synchronize()
    assert_attn_close(out, want, f"prefill batch {batch} heads {hq}/{hkv} q<= {q_hi} prefix {prefix_fraction}")
    assert torch.equal(run(), out)
