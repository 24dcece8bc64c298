"""Paged decode attention on the GPU, through the C ABI, against the fp32 oracle."""
import pytest
import torch

import oracle
from nanovllm_amd import paged_decode_attention
from nanovllm_amd import synthetic
from nanovllm_amd.context import DecodePlan
from helpers import assert_attn_close, bits

pytestmark = pytest.mark.gpu


def _gpu(case, dev, tables=None):
    t = case.block_tables if tables is None else tables
    out = paged_decode_attention(case.q.to(dev), case.k_cache.to(dev), case.v_cache.to(dev),
                                 case.context_lens.to(dev), t.to(dev), case.scale)
    torch.cuda.synchronize()
    return out


def _oracle(case):
    return oracle.paged_decode_attention(case.q, case.k_cache, case.v_cache, case.context_lens,
                                         case.block_tables, case.scale, "fp32")


def test_decode_config2(dev):
    """batch 64, 16 q / 8 kv heads, head_dim 128, ctx U[100,2048], 1024-block pool."""
    case = synthetic.decode_case(seed=0)
    out = _gpu(case, dev)
    assert out.shape == (64, 1, 16, 128) and out.dtype == torch.bfloat16
    assert_attn_close(out, _oracle(case), "config 2")


@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 8), (16, 2), (8, 1), (24, 8), (40, 8), (12, 2), (7, 1),   # groups 4 1 8 8 3 5 6 7
                                    (6, 3), (12, 6), (10, 5), (12, 12)])                                     # kv heads that are no multiple of 4: 1 or 2 heads side by side
def test_decode_gqa_groups(dev, hq, hkv):
    case = synthetic.decode_case(seed=hq * 10 + hkv, batch=9, num_heads=hq, num_kv_heads=hkv, num_blocks=64,
                                 ctx_lo=1, ctx_hi=1200)
    assert_attn_close(_gpu(case, dev), _oracle(case), f"gqa {hq}/{hkv}")


@pytest.mark.parametrize("block_size", [512, 1024, 4096])
def test_decode_larger_kv_blocks(dev, block_size):
    """KV blocks of 256 * 2^k tokens (nanovllm/config.py:22 allows multiples of 256)."""
    case = synthetic.decode_case(seed=block_size, batch=7, num_blocks=max(8, 16384 // block_size * 2), ctx_lo=1,
                                 ctx_hi=3000, block_size=block_size)
    assert case.k_cache.shape[1] == block_size
    assert_attn_close(_gpu(case, dev), _oracle(case), f"block size {block_size}")


def test_decode_edge_context_lengths(dev):
    lens = [0, 1, 2, 63, 64, 65, 255, 256, 257, 511, 512, 513, 1024, 0, 3]
    case = synthetic.decode_case(seed=7, num_blocks=64, context_lens=lens)
    out = _gpu(case, dev)
    want = _oracle(case)
    assert_attn_close(out, want, "edge lens")
    assert not out[0].any() and not out[13].any()              # context_len 0 -> zeros
    # one key: the output is exactly that V row (bf16 round trip of fp32 is the identity)
    blk = int(case.block_tables[1, 0])
    assert torch.equal(bits(out[1, 0, 0]), bits(case.v_cache[blk, 0, 0]))
    assert torch.equal(bits(out[1, 0, 1]), bits(case.v_cache[blk, 0, 0]))     # heads 0,1 -> kv head 0
    assert torch.equal(bits(out[1, 0, 15]), bits(case.v_cache[blk, 0, 7]))


def test_decode_ignores_stale_and_padded_table_entries(dev):
    """Only entries j < ceil(ctx/256) may be dereferenced: the rest may be -1, stale ids of
    other sequences, or out-of-range garbage (graph replays never clear the table)."""
    case = synthetic.decode_case(seed=8, batch=12, num_blocks=64, ctx_lo=1, ctx_hi=1500)
    base = _gpu(case, dev)
    wide = torch.full((12, 16), -1, dtype=torch.int32)
    wide[:, : case.block_tables.shape[1]] = case.block_tables
    need = (case.context_lens + 255) // 256
    g = torch.Generator().manual_seed(1)
    for b in range(12):
        n = int(need[b])
        junk = torch.randint(0, 64, (16 - n,), generator=g, dtype=torch.int32)
        junk[::3] = 1 << 30
        junk[1::3] = -5
        wide[b, n:] = junk
    out = _gpu(case, dev, wide)
    assert torch.equal(bits(out), bits(base))
    assert_attn_close(out, _oracle(case), "stale tables")


def test_decode_invariants(dev):
    case = synthetic.decode_case(seed=9, batch=8, num_blocks=48, ctx_lo=200, ctx_hi=1100)
    out = _gpu(case, dev)
    # V == 1 -> out == 1
    ones = synthetic.DecodeCase(case.q, case.k_cache, torch.ones_like(case.v_cache), case.context_lens,
                                case.block_tables, case.scale)
    o1 = _gpu(ones, dev).float().cpu()
    assert (o1 - 1).abs().max() < 1e-2
    # renaming physical blocks changes nothing, bit for bit
    perm = torch.randperm(48, generator=torch.Generator().manual_seed(2))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(48)
    t2 = torch.where(case.block_tables >= 0, inv[case.block_tables.clamp_min(0).long()].to(torch.int32),
                     case.block_tables)
    moved = synthetic.DecodeCase(case.q, case.k_cache[perm], case.v_cache[perm], case.context_lens, t2, case.scale)
    assert torch.equal(bits(_gpu(moved, dev)), bits(out))
    # garbage beyond context_len inside the last block is never used
    kc, vc = case.k_cache.clone(), case.v_cache.clone()
    for b in range(8):
        n = int(case.context_lens[b])
        last = int(case.block_tables[b, (n - 1) // 256])
        kc[last, n % 256 if n % 256 else 256:] = float("nan")
        vc[last, n % 256 if n % 256 else 256:] = float("inf")
    dirty = synthetic.DecodeCase(case.q, kc, vc, case.context_lens, case.block_tables, case.scale)
    assert torch.equal(bits(_gpu(dirty, dev)), bits(out))


def test_decode_long_context_many_splits(dev):
    """Qwen3-8B geometry (32/8 heads), 65-wide tables, contexts up to 16384."""
    lens = [16384, 4096, 9001, 12345]
    case = synthetic.decode_case(seed=11, num_heads=32, num_kv_heads=8, num_blocks=180, context_lens=lens)
    assert_attn_close(_gpu(case, dev), _oracle(case), "long ctx")


def test_decode_q_as_4d_and_strided(dev):
    case = synthetic.decode_case(seed=12, batch=5, num_blocks=32, ctx_lo=10, ctx_hi=700)
    qkv = torch.zeros(5, 16 * 128 + 2 * 8 * 128, dtype=torch.bfloat16)
    qkv[:, : 16 * 128] = case.q.reshape(5, -1)
    qd = qkv.to(dev)[:, : 16 * 128].view(5, 16, 128)            # row stride 4096
    out = paged_decode_attention(qd.unsqueeze(1), case.k_cache.to(dev), case.v_cache.to(dev),
                                 case.context_lens.to(dev), case.block_tables.to(dev), case.scale)
    torch.cuda.synchronize()
    assert_attn_close(out, _oracle(case), "strided q")


def test_decode_partials_are_fresh_across_calls(dev):
    """Split partials travel between XCDs through memory.  Two different inputs of the same shape
    use the same partial rows, so a stale read would surface as a mismatch when they alternate."""
    cases = [synthetic.decode_case(seed=40 + i, batch=24, num_blocks=256, ctx_lo=1500, ctx_hi=1600) for i in range(2)]
    cases[1].context_lens[:] = cases[0].context_lens            # same stage list, same split, other values
    cases[1] = synthetic.DecodeCase(cases[1].q, cases[1].k_cache, cases[1].v_cache, cases[0].context_lens,
                                    cases[0].block_tables, cases[1].scale)
    dev_in = [(c.q.to(dev), c.k_cache.to(dev), c.v_cache.to(dev), c.context_lens.to(dev), c.block_tables.to(dev))
              for c in cases]
    good = []
    for c, d in zip(cases, dev_in):
        out = paged_decode_attention(*d, c.scale)
        torch.cuda.synchronize()
        assert_attn_close(out, _oracle(c), "alternating")
        good.append(out.clone())
    for it in range(300):
        i = it & 1
        out = paged_decode_attention(*dev_in[i], cases[i].scale)
        assert torch.equal(out, good[i]), f"iteration {it}"


@pytest.mark.parametrize("shape", ["few_stages", "edge_lens", "many_splits", "config2"])
def test_decode_plan_reuse_is_bit_identical(dev, shape):
    """The layers of one decode step share context_lens and block_tables: the first call derives
    the work split, the others reuse it from the workspace.  Both paths run the same arithmetic in
    the same order, so the outputs are equal bit for bit, whatever q and caches a layer brings."""
    if shape == "few_stages":         # fewer stages than workers: one stage per worker, idle workers
        kw = dict(batch=5, num_blocks=64, ctx_lo=1, ctx_hi=300)
    elif shape == "edge_lens":
        kw = dict(num_blocks=64, context_lens=[0, 1, 2, 63, 64, 65, 255, 256, 257, 511, 512, 513, 1024, 0, 3])
    elif shape == "many_splits":
        kw = dict(batch=3, num_blocks=256, ctx_lo=9000, ctx_hi=12000)
    else:
        kw = {}
    layers = [synthetic.decode_case(seed=60 + i, **kw) for i in range(3)]
    ctx = layers[0].context_lens.to(dev)
    tables = layers[0].block_tables.to(dev)
    dev_in = [(c.q.to(dev), c.k_cache.to(dev), c.v_cache.to(dev)) for c in layers]
    alone = [paged_decode_attention(*d, ctx, tables, layers[0].scale).clone() for d in dev_in]
    want = oracle.paged_decode_attention(layers[0].q, layers[0].k_cache, layers[0].v_cache, layers[0].context_lens,
                                         layers[0].block_tables, layers[0].scale, "fp32")
    assert_attn_close(alone[0], want, shape)
    for step in range(2):                                  # a second step rebuilds over the old records
        plan = DecodePlan()
        for d, good in zip(dev_in, alone):
            out = paged_decode_attention(*d, ctx, tables, layers[0].scale, plan=plan)
            assert torch.equal(out, good), (shape, step)
    # a different batch after a plan was built: the next build must not see stale records
    other = synthetic.decode_case(seed=70, batch=40, num_blocks=128, ctx_lo=1, ctx_hi=900)
    od = (other.q.to(dev), other.k_cache.to(dev), other.v_cache.to(dev), other.context_lens.to(dev),
          other.block_tables.to(dev))
    o_alone = paged_decode_attention(*od, other.scale).clone()
    plan = DecodePlan()
    for _ in range(3):
        assert torch.equal(paged_decode_attention(*od, other.scale, plan=plan), o_alone)


def test_decode_plan_survives_another_batch_in_between(dev):
    """All decode calls of a device share one workspace, the stored work split included.  A call on
    another batch between a plan's first call and a later one overwrites the split; the later call
    must notice and derive its own again instead of following the other batch's records."""
    a = synthetic.decode_case(seed=90, batch=24, num_blocks=128, ctx_lo=1, ctx_hi=1200)
    b = synthetic.decode_case(seed=91, batch=9, num_blocks=128, ctx_lo=300, ctx_hi=3000)
    da = (a.q.to(dev), a.k_cache.to(dev), a.v_cache.to(dev), a.context_lens.to(dev), a.block_tables.to(dev))
    db = (b.q.to(dev), b.k_cache.to(dev), b.v_cache.to(dev), b.context_lens.to(dev), b.block_tables.to(dev))
    want_a = paged_decode_attention(*da, a.scale).clone()
    want_b = paged_decode_attention(*db, b.scale).clone()
    assert_attn_close(want_a, _oracle(a), "batch a")
    plan_a, plan_b = DecodePlan(), DecodePlan()
    assert torch.equal(paged_decode_attention(*da, a.scale, plan=plan_a), want_a)      # builds
    assert torch.equal(paged_decode_attention(*db, b.scale, plan=plan_b), want_b)      # builds over it
    assert torch.equal(paged_decode_attention(*da, a.scale, plan=plan_a), want_a)      # must rebuild
    assert torch.equal(paged_decode_attention(*da, a.scale, plan=plan_a), want_a)      # reuses its own again
    assert torch.equal(paged_decode_attention(*db, b.scale), want_b)                   # a call without a plan builds too
    assert torch.equal(paged_decode_attention(*da, a.scale, plan=plan_a), want_a)


def test_decode_batch_above_one_launch(dev):
    """More than 1024 sequences run as two launches sharing the workspace; a stored work split is
    then never reused (each launch overwrites it), with or without a plan object."""
    case = synthetic.decode_case(seed=81, batch=1100, num_heads=2, num_kv_heads=1, num_blocks=1200, ctx_lo=1, ctx_hi=256)
    d = (case.q.to(dev), case.k_cache.to(dev), case.v_cache.to(dev), case.context_lens.to(dev),
         case.block_tables.to(dev))
    out = paged_decode_attention(*d, case.scale).clone()
    assert_attn_close(out, _oracle(case), "batch 1100")
    plan = DecodePlan()
    for _ in range(3):
        assert torch.equal(paged_decode_attention(*d, case.scale, plan=plan), out)


def test_decode_plan_rejects_a_different_batch(dev):
    case = synthetic.decode_case(seed=80, batch=6, num_blocks=64, ctx_lo=1, ctx_hi=600)
    d = (case.q.to(dev), case.k_cache.to(dev), case.v_cache.to(dev), case.context_lens.to(dev),
         case.block_tables.to(dev))
    plan = DecodePlan()
    paged_decode_attention(*d, case.scale, plan=plan)
    with pytest.raises(ValueError):
        paged_decode_attention(d[0][:4], d[1], d[2], d[3][:4], d[4][:4], case.scale, plan=plan)


def test_decode_config5_full_size(dev):
    """The long-context stress shape at full size: batch 128, 32 q / 8 kv heads, contexts
    U[4096,16384], blocks scattered over a 5.4 GB pool.  Too big for the oracle as a whole, so:
    three sequences are re-stated as a small case (their pages gathered, tables renumbered) and
    checked against the fp32 oracle, both as rows of the big launch and launched alone (a
    different split of the work); the output does not depend on the physical placement of the
    blocks (bit for bit); V == 1 gives 1."""
    g = torch.Generator().manual_seed(5)
    ctx = torch.randint(4096, 16385, (128,), generator=g, dtype=torch.int32)
    need = int(((ctx + 255) // 256).sum())
    tables = synthetic.decode_tables(ctx.tolist(), need + 8, g)
    gd = torch.Generator(device=dev).manual_seed(6)
    kc = torch.empty((need + 8, 256, 8, 128), device=dev, dtype=torch.bfloat16).normal_(generator=gd)
    vc = torch.empty((need + 8, 256, 8, 128), device=dev, dtype=torch.bfloat16).normal_(generator=gd)
    q = torch.randn((128, 32, 128), generator=g).to(torch.bfloat16)
    scale = 128 ** -0.5
    out = paged_decode_attention(q.to(dev), kc, vc, ctx.to(dev), tables.to(dev), scale)
    torch.cuda.synchronize()
    assert out.shape == (128, 1, 32, 128)
    pick = [0, 57, 127, int(ctx.argmax()), int(ctx.argmin())]
    # the picked sequences as a case of their own: pages gathered to a private pool
    blocks = [tables[b, : (int(ctx[b]) + 255) // 256].long() for b in pick]
    flat = torch.cat(blocks)
    small_k, small_v = kc[flat.to(dev)].cpu(), vc[flat.to(dev)].cpu()
    small_t = torch.full((len(pick), tables.shape[1]), -1, dtype=torch.int32)
    at = 0
    for i, blk in enumerate(blocks):
        small_t[i, : len(blk)] = torch.arange(at, at + len(blk), dtype=torch.int32)
        at += len(blk)
    want = oracle.paged_decode_attention(q[pick], small_k, small_v, ctx[pick], small_t, scale, "fp32")
    assert_attn_close(out[pick], want, "config 5 rows vs oracle")
    alone = paged_decode_attention(q[pick].to(dev), small_k.to(dev), small_v.to(dev), ctx[pick].to(dev),
                                   small_t.to(dev), scale)
    assert_attn_close(alone, want, "config 5 rows alone")
    # physical placement: reverse the pool
    rev = torch.arange(need + 7, -1, -1)
    t2 = torch.where(tables >= 0, (need + 7 - tables.clamp_min(0)).to(torch.int32), tables)
    out2 = paged_decode_attention(q.to(dev), kc[rev.to(dev)], vc[rev.to(dev)], ctx.to(dev), t2.to(dev), scale)
    assert torch.equal(bits(out2), bits(out))
    del out2
    ones = paged_decode_attention(q.to(dev), kc, torch.ones_like(vc), ctx.to(dev), tables.to(dev), scale)
    assert (ones.float() - 1).abs().max().item() < 1e-2


@pytest.mark.parametrize("batch,hq,hkv", [(32, 16, 8), (31, 16, 8), (64, 32, 8), (40, 8, 8), (300, 16, 8), (33, 8, 8)])
def test_decode_ragged_batches_share_a_workspace(dev, batch, hq, hkv):
    """Ragged contexts with empty, one-token and very short sequences beside long ones, batch sizes
    from few to many (sequence, kv head) pairs per worker, several decode steps in a row on the one
    workspace of the device (a build and two reuses of the work split each), against the fp32
    oracle; every call of a geometry returns the same bits."""
    g = torch.Generator().manual_seed(batch * 100 + hq)
    lens = torch.randint(1, 3000, (batch,), generator=g)
    lens[::7] = torch.randint(1, 40, (len(lens[::7]),), generator=g)          # very short ones
    lens[3] = 0
    lens[5] = 1
    need = int(((lens + 255) // 256).sum()) + 4
    case = synthetic.decode_case(seed=batch + hq, num_heads=hq, num_kv_heads=hkv, num_blocks=need, context_lens=lens.tolist())
    want = _oracle(case)
    q, kc, vc, cl, bt = (t.to(dev) for t in (case.q, case.k_cache, case.v_cache, case.context_lens, case.block_tables))
    outs = []
    for _ in range(3):
        plan = DecodePlan()
        for _layer in range(3):                                  # one build, two reuses
            outs.append(paged_decode_attention(q, kc, vc, cl, bt, case.scale, plan=plan).clone())
    torch.cuda.synchronize()
    for o in outs:
        assert_attn_close(o, want, f"batch {batch}")
    for o in outs[1:]:
        assert torch.equal(bits(o), bits(outs[0]))
    assert not outs[0][3].any()
