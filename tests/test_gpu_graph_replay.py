"""The hot path captured in a hipGraph and replayed with new contents, against eager calls and the oracle.

nanovllm/engine/model_runner.py:215-250 captures one decode step per batch bucket over STATIC tensors and
replays it with new contents (:197-204): shapes and pointers never change, values do, block-table columns past
the current width keep stale ids and padded rows carry context length 0 and slot -1.  Here one graph holds what a
two-layer decode step needs from the library -- scatter, decode attention that derives the work split, decode
attention of a second "layer" that reuses it, the fused norm + rotary + cache write, and the sampler -- and is
replayed several times, with eager work and synchronisation in between, each replay on freshly drawn contents.
Every replay must be bit-identical to the same calls made eagerly on the same contents, bit-exact against the
oracle's scatter, and within the attention tolerance of the fp32 oracle.
"""
import pytest
import torch

import oracle
from nanovllm_amd import paged_decode_attention, sample, store_kvcache, synthetic
from nanovllm_amd.context import DecodePlan
from nanovllm_amd.engine import layers
from helpers import assert_attn_close, bits

pytestmark = pytest.mark.gpu

B, HQ, HKV, D, WIDTH, BLOCKS, VOCAB = 24, 16, 8, 128, 6, 160, 20000


def _draw(seed, dev, live):
    """Contents of one decode step: `live` sequences, the other rows padded the way the runner pads a bucket."""
    g = torch.Generator().manual_seed(seed)
    ctx = torch.zeros(B, dtype=torch.int32)
    ctx[:live] = torch.randint(1, WIDTH * 256 + 1, (live,), generator=g, dtype=torch.int32)
    tables = torch.randint(0, BLOCKS, (B, WIDTH), generator=g, dtype=torch.int32)      # stale ids everywhere ...
    fresh = synthetic.decode_tables(ctx[:live].tolist(), BLOCKS, g, width=WIDTH)
    need = (ctx[:live].to(torch.int64) + 255) // 256
    for i in range(live):
        tables[i, : int(need[i])] = fresh[i, : int(need[i])]                            # ... except where a sequence has keys
    slots = torch.full((B,), -1, dtype=torch.int32)
    last = ctx[:live].to(torch.int64) - 1
    slots[:live] = (tables[torch.arange(live), last // 256].to(torch.int64) * 256 + last % 256).to(torch.int32)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(torch.bfloat16)
    return dict(ctx=ctx, tables=tables, slots=slots, q=rnd(B, HQ, D), k=rnd(B, HKV, D), v=rnd(B, HKV, D),
                qkv=rnd(B, (HQ + 2 * HKV) * D), pos=(ctx.to(torch.int64) - 1).clamp_min(0),
                logits=(torch.randn(B, VOCAB, generator=g) * 2).to(torch.bfloat16))


def _step(st, caches, rope, w, plan_pair):
    """The library calls of a two-layer decode step over the tensors in `st`; returns everything they produce."""
    (kc0, vc0), (kc1, vc1) = caches
    store_kvcache(st["k"], st["v"], kc0, vc0, st["slots"])
    plan = DecodePlan() if plan_pair else None
    o0 = paged_decode_attention(st["q"], kc0, vc0, st["ctx"], st["tables"], D ** -0.5, plan=plan)
    q1, k1, _ = layers.qk_norm_rope(st["qkv"], st["pos"], w, w, rope, HQ, HKV, D, 1e-6, kv_store=(kc1, vc1, st["slots"]))
    o1 = paged_decode_attention(q1, kc1, vc1, st["ctx"], st["tables"], D ** -0.5, plan=plan)   # second layer: reuses the split
    tok = sample(st["logits"], st["temps"], None, seed=11, offset=5)
    return o0, o1, q1, k1, tok


@pytest.mark.parametrize("shared_split", [True, False])
def test_graph_replays_match_eager_calls_and_the_oracle(dev, shared_split):
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(1)
    pool = [torch.randn(BLOCKS, 256, HKV, D, generator=g).to(torch.bfloat16) for _ in range(4)]
    caches = [(pool[0].to(dev), pool[1].to(dev)), (pool[2].to(dev), pool[3].to(dev))]
    rope = layers.build_rope_cache(D, WIDTH * 256, 1e6, dev)
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16).to(dev)
    first = _draw(100, dev, B)
    st = {k: v.to(dev) for k, v in first.items()}
    st["temps"] = torch.full((B,), 0.7, device=dev)
    st["temps"][::6] = 0.0                                             # some greedy rows

    _step(st, caches, rope, w, shared_split)                           # eager warm-up: sizes the decode workspace
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = _step(st, caches, rope, w, shared_split)
    torch.cuda.synchronize()

    for r, live in enumerate([B, 7, 19, 1]):                           # smaller batches leave padded rows and stale tables behind
        new = _draw(200 + r, dev, live)
        for name, value in new.items():
            st[name].copy_(value.to(dev))
        before = [(kc.clone(), vc.clone()) for kc, vc in caches]       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        after = [(kc.clone(), vc.clone()) for kc, vc in caches]
        # the same calls, eagerly, from the same cache state
        for (kc, vc), (bk, bv) in zip(caches, before):
            kc.copy_(bk)
            vc.copy_(bv)
        want = _step(st, caches, rope, w, shared_split)
        torch.cuda.synchronize()
        for name, a, b in zip(("o0", "o1", "q1", "k1", "tokens"), got, want):
            assert torch.equal(a, b), f"replay {r} ({live} live rows): {name} differs from the eager call"
        for (kc, vc), (ak, av) in zip(caches, after):
            assert torch.equal(kc, ak) and torch.equal(vc, av), f"replay {r}: cache differs from the eager call"
        # layer 0 against the oracle: scatter bit-exact, attention within tolerance, padded rows zero
        ek, ev = before[0][0].cpu(), before[0][1].cpu()
        oracle.store_kvcache(new["k"], new["v"], ek, ev, new["slots"])
        assert torch.equal(bits(after[0][0]), bits(ek)) and torch.equal(bits(after[0][1]), bits(ev))
        ref = oracle.paged_decode_attention(new["q"][:live], ek, ev, new["ctx"][:live], new["tables"][:live], D ** -0.5, "fp32")
        assert_attn_close(got[0][:live], ref, f"replay {r} layer 0")
        assert not got[0][live:].any() and not got[1][live:].any(), "rows without keys must be zero"
        greedy = new["logits"].float().argmax(-1)
        assert torch.equal(got[4].cpu()[::6], greedy[::6])


def test_attention_module_under_the_reference_capture_pattern(dev):
    """nanovllm/engine/model_runner.py:229-237 installs ONE context per batch size, runs the model once
    eagerly (warm-up) and once more under graph capture, then replays the graph on new contents of the
    same tensors.  Three Attention layers driven that way, with no plan supplied by the runner: the
    layers share a work split on their own (the first derives it, the others reuse it), the captured
    layers must not lean on the split the warm-up run left behind, and every replay must equal the
    eager result of a fresh context and stay within tolerance of the oracle."""
    import nanovllm_amd as nva
    from nanovllm_amd.context import get_context
    g = torch.Generator().manual_seed(5)
    n_layers = 3
    pools = [(torch.randn(BLOCKS, 256, HKV, D, generator=g).to(torch.bfloat16).to(dev),
              torch.randn(BLOCKS, 256, HKV, D, generator=g).to(torch.bfloat16).to(dev)) for _ in range(n_layers)]
    attn = []
    for kc, vc in pools:
        layer = nva.Attention(HQ, D, D ** -0.5, HKV)
        layer.k_cache, layer.v_cache = kc, vc
        attn.append(layer)
    st = {k: v.to(dev) for k, v in _draw(300, dev, B).items()}
    qs = [torch.randn(B, HQ, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(n_layers)]

    def forward():
        return [layer(q, st["k"], st["v"]).clone() for layer, q in zip(attn, qs)]

    nva.set_context(False, slot_mapping=st["slots"], context_lens=st["ctx"], block_tables=st["tables"])
    forward()                                                          # warm-up under the context ...
    warm_plan = get_context().decode_plan
    assert warm_plan is not None and not warm_plan.capturing           # ... whose layers shared a split
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):                                      # ... and capture under the same one
        captured = forward()
    assert get_context().decode_plan is not warm_plan and get_context().decode_plan.capturing
    nva.reset_context()
    torch.cuda.synchronize()
    for r, live in enumerate([B, 5, 17]):
        new = _draw(400 + r, dev, live)
        for name, value in new.items():
            st[name].copy_(value.to(dev))
        before = [(kc.clone(), vc.clone()) for kc, vc in pools]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        for (kc, vc), (bk, bv) in zip(pools, before):
            kc.copy_(bk)
            vc.copy_(bv)
        nva.set_context(False, slot_mapping=st["slots"], context_lens=st["ctx"], block_tables=st["tables"])
        want = forward()                                               # a fresh context: builds, then reuses
        nva.reset_context()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {r}: layer {i} differs from the eager call"
        ek, ev = before[0][0].cpu(), before[0][1].cpu()
        oracle.store_kvcache(new["k"], new["v"], ek, ev, new["slots"])
        ref = oracle.paged_decode_attention(qs[0][:live].cpu(), ek, ev, new["ctx"][:live], new["tables"][:live], D ** -0.5, "fp32")
        assert_attn_close(got[0][:live, 0], ref, f"replay {r} layer 0")
