"""Fused glue kernels (RMSNorm, q/k-norm + rotary, SwiGLU gate) against oracle/glue.py.

The kernels keep the reference's rounding points, so results agree to the last bf16 bit
except where a different fp32 summation order moves a value across a rounding boundary:
the tests allow one bf16 ulp on a small fraction of the elements (two on a handful)."""
import pytest
import torch

from oracle import glue
from nanovllm_amd.engine import layers

pytestmark = pytest.mark.gpu


def assert_bf16_close(got, want, what, max_frac=0.02):
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all()
    ulp = want.abs().clamp_min(1e-30) * 2.0 ** -7          # one bf16 step at the value's magnitude
    diff = (got - want).abs()
    # the value is rounded twice (after the normalisation and after the weight multiply), so a
    # one-ulp difference of the first rounding can become two ulps at the output
    assert bool((diff <= ulp * 2.02 + 1e-30).all()), f"{what}: max diff {float(diff.max())} exceeds two bf16 ulps"
    assert float((diff > ulp * 1.01).float().mean()) <= 1e-4, f"{what}: too many two-ulp differences"
    frac = float((diff > 0).float().mean())
    assert frac <= max_frac, f"{what}: {frac:.4f} of the elements differ"


@pytest.mark.parametrize("rows,hidden", [(1, 1024), (256, 1024), (77, 4096), (5, 128), (3, 1000), (4097, 1024)])
def test_rms_norm_and_add_rms_norm(dev, rows, hidden):
    g = torch.Generator().manual_seed(rows + hidden)
    x = (torch.randn(rows, hidden, generator=g) * 3).to(torch.bfloat16)
    r = torch.randn(rows, hidden, generator=g).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    out = layers.rms_norm(x.to(dev), w.to(dev), 1e-6)
    assert_bf16_close(out, glue.rms_norm(x, w, 1e-6), "rms_norm")
    out2, res2 = layers.add_rms_norm(x.to(dev), r.to(dev), w.to(dev), 1e-6)
    want, want_res = glue.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(res2.cpu().view(torch.int16), want_res.view(torch.int16))     # the sum is exact
    assert_bf16_close(out2, want, "add_rms_norm")


@pytest.mark.parametrize("batch,total,hidden", [(29, 16384, 1024), (4, 700, 4096), (1, 1, 1024), (7, 50, 1000)])
def test_gather_last_rms_norm_is_the_full_norm_at_the_last_rows(dev, batch, total, hidden):
    """The final norm on the last token of every sequence only (what the LM head of a prefill step
    reads) against the oracle's full norm followed by the gather, with and without a residual; and
    bit for bit the rows the full-size kernel produces."""
    g = torch.Generator().manual_seed(batch * 31 + hidden)
    x = (torch.randn(total, hidden, generator=g) * 3).to(torch.bfloat16)
    r = torch.randn(total, hidden, generator=g).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    cuts = torch.sort(torch.randperm(total - 1, generator=g)[: batch - 1] + 1).values if batch > 1 else torch.empty(0, dtype=torch.long)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([total])]).to(torch.int32)
    got = layers.gather_last_rms_norm(x.to(dev), r.to(dev), cu.to(dev), w.to(dev), 1e-6)
    assert got.shape == (batch, hidden)
    assert_bf16_close(got, glue.last_token_norm(x, r, cu, w, 1e-6), "gather + add + norm")
    full, _ = layers.add_rms_norm(x.to(dev), r.to(dev), w.to(dev), 1e-6)
    assert torch.equal(got, full[(cu[1:] - 1).long().to(dev)])
    got = layers.gather_last_rms_norm(x.to(dev), None, cu.to(dev), w.to(dev), 1e-6)
    assert_bf16_close(got, glue.last_token_norm(x, None, cu, w, 1e-6), "gather + norm")


def test_gather_last_rms_norm_empty_spans_and_strided_rows(dev):
    """An empty query span picks the previous sequence's last row and an empty FIRST span wraps to
    the last row of the tensor, as the reference's ``x[cu_seqlens_q[1:] - 1]`` does; rows may be
    strided views; a bound beyond the tensor is clamped instead of read out of bounds."""
    g = torch.Generator().manual_seed(5)
    wide = torch.randn(40, 2048, generator=g).to(torch.bfloat16)
    r = torch.randn(40, 1024, generator=g).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(1024, generator=g)).to(torch.bfloat16)
    x = wide[:, 512:1536]
    cu = torch.tensor([0, 0, 13, 13, 40], dtype=torch.int32)
    got = layers.gather_last_rms_norm(wide.to(dev)[:, 512:1536], r.to(dev), cu.to(dev), w.to(dev), 1e-6)
    assert_bf16_close(got, glue.last_token_norm(x, r, cu, w, 1e-6), "empty spans")
    assert torch.equal(got[1], got[2]) and not torch.equal(got[0], got[1])
    beyond = torch.tensor([0, 13, 900], dtype=torch.int32)
    got = layers.gather_last_rms_norm(wide.to(dev)[:, 512:1536], r.to(dev), beyond.to(dev), w.to(dev), 1e-6)
    want = glue.last_token_norm(x, r, torch.tensor([0, 13, 40], dtype=torch.int32), w, 1e-6)
    assert_bf16_close(got, want, "clamped bound")


def test_rms_norm_strided_rows(dev):
    g = torch.Generator().manual_seed(9)
    wide = torch.randn(16, 2048, generator=g).to(torch.bfloat16)
    w = torch.ones(1024, dtype=torch.bfloat16)
    out = layers.rms_norm(wide.to(dev)[:, 512:1536], w.to(dev), 1e-6)
    assert_bf16_close(out, glue.rms_norm(wide[:, 512:1536], w, 1e-6), "strided")


@pytest.mark.parametrize("n,hq,hkv", [(1, 16, 8), (256, 16, 8), (1000, 32, 8), (3, 4, 1)])
def test_qk_norm_rope(dev, n, hq, hkv):
    g = torch.Generator().manual_seed(n)
    d = 128
    qkv = torch.randn(n, (hq + 2 * hkv) * d, generator=g).to(torch.bfloat16)
    qw = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16)
    kw = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16)
    pos = torch.randint(0, 4096, (n,), generator=g)
    cache = glue.build_rope_cache(d, 4096, 1e6)
    cache_d = layers.build_rope_cache(d, 4096, 1e6, dev)
    assert (cache_d.cpu() - cache).abs().max() < 1e-3         # table built on the device: pow() differs in the last ulp and positions up to 4095 amplify it
    qkv_d = qkv.to(dev)
    q, k, v = layers.qk_norm_rope(qkv_d, pos.to(dev), qw.to(dev), kw.to(dev), cache.to(dev), hq, hkv, d, 1e-6)
    wq, wk, wv = glue.qk_norm_rope(qkv, pos, qw, kw, cache, hq, hkv, d, 1e-6)
    assert q.is_contiguous() and k.is_contiguous()
    assert v.data_ptr() == qkv_d.data_ptr() + (hq + hkv) * d * 2 and (n == 1 or v.stride(0) == (hq + 2 * hkv) * d)
    assert torch.equal(v.cpu().view(torch.int16), wv.contiguous().view(torch.int16))
    # the rotation subtracts nearly equal products: compare against the value scale, not per element
    for got, want, name in ((q, wq, "q"), (k, wk, "k")):
        diff = (got.float().cpu() - want.float()).abs()
        assert float(diff.max()) <= 2.0 ** -6 * float(want.float().abs().max()), name
        assert float(diff.mean()) <= 1e-3, name


@pytest.mark.parametrize("rows,inter", [(1, 3072), (256, 3072), (50, 12288), (7, 8)])
def test_silu_and_mul(dev, rows, inter):
    g = torch.Generator().manual_seed(inter)
    x = (torch.randn(rows, 2 * inter, generator=g) * 2).to(torch.bfloat16)
    out = layers.silu_and_mul(x.to(dev))
    assert_bf16_close(out, glue.silu_and_mul(x), "silu_and_mul", max_frac=0.01)


def test_qk_norm_rope_fused_scatter_matches_store_kvcache(dev):
    """The fused kernel writes to the cache exactly what store_kvcache writes from its outputs."""
    import nanovllm_amd as nva
    g = torch.Generator().manual_seed(21)
    n, hq, hkv, d = 300, 16, 8, 128
    qkv = torch.randn(n, (hq + 2 * hkv) * d, generator=g).to(torch.bfloat16).to(dev)
    w = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16).to(dev)
    pos = torch.randint(0, 4096, (n,), generator=g).to(dev)
    cache = layers.build_rope_cache(d, 4096, 1e6, dev)
    slots = torch.randperm(4 * 256, generator=g)[:n].to(torch.int32)
    slots[::7] = -1
    slots = slots.to(dev)
    kc1, vc1 = (torch.zeros(4, 256, hkv, d, dtype=torch.bfloat16, device=dev) for _ in range(2))
    kc2, vc2 = torch.zeros_like(kc1), torch.zeros_like(vc1)
    q1, k1, v1 = layers.qk_norm_rope(qkv, pos, w, w, cache, hq, hkv, d, 1e-6, kv_store=(kc1, vc1, slots))
    q2, k2, v2 = layers.qk_norm_rope(qkv, pos, w, w, cache, hq, hkv, d, 1e-6)
    nva.store_kvcache(k2, v2, kc2, vc2, slots)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2)
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2) and bool(kc1.any()) and bool(vc1.any())


@pytest.mark.parametrize("hq,hkv", [(16, 8), (32, 8)])
def test_fused_scatter_is_bit_exact_against_the_oracle_scatter(dev, hq, hkv):
    """The scatter the engine really runs -- nva_qk_norm_rope with cache pointers -- on the slot
    mapping of the scatter benchmark configuration (4096 tokens into 512 blocks x 256 slots, 5 %
    skipped, value rows strided inside the fused qkv buffer), against oracle.store_kvcache:
      * V cache bit-exact (the rows are copied unchanged);
      * K cache bit-exact against the oracle scatter of the key rows the kernel returned (slot
        indexing), and those rows against the oracle's norm + rope to the glue tolerance (most bits equal);
      * every slot that was not addressed is still zero."""
    import oracle
    from nanovllm_amd import synthetic
    case = synthetic.scatter_case(seed=0)
    n, d = case.slot_mapping.numel(), 128
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn(n, (hq + 2 * hkv) * d, generator=g).to(torch.bfloat16)
    qw = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16)
    kw = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16)
    pos = torch.randint(0, 4096, (n,), generator=g)
    rope = glue.build_rope_cache(d, 4096, 1e6)
    slots = case.slot_mapping
    kc = torch.zeros(512, 256, hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    q, k, v = layers.qk_norm_rope(qkv.to(dev), pos.to(dev), qw.to(dev), kw.to(dev), rope.to(dev), hq, hkv, d, 1e-6,
                                  kv_store=(kc, vc, slots.to(dev)))
    torch.cuda.synchronize()
    wq, wk, wv = glue.qk_norm_rope(qkv, pos, qw, kw, rope, hq, hkv, d, 1e-6)
    ek, ev = torch.zeros(512, 256, hkv, d, dtype=torch.bfloat16), torch.zeros(512, 256, hkv, d, dtype=torch.bfloat16)
    oracle.store_kvcache(wk.contiguous(), wv, ek, ev, slots)
    as_bits = lambda t: t.cpu().contiguous().view(torch.int16)
    assert torch.equal(as_bits(vc), as_bits(ev))                                  # values: bit-exact
    ek2, ev2 = torch.zeros_like(ek), torch.zeros_like(ev)
    oracle.store_kvcache(k.cpu(), v.cpu(), ek2, ev2, slots)
    assert torch.equal(as_bits(kc), as_bits(ek2)) and torch.equal(as_bits(vc), as_bits(ev2))   # slot indexing: bit-exact
    same = float((as_bits(kc) == as_bits(ek)).float().mean())
    assert same >= 0.97, same                                                      # keys: the oracle's bits almost everywhere
    diff = (kc.cpu().float() - ek.float()).abs()
    assert float(diff.max()) <= 2.0 ** -6 * float(ek.float().abs().max())
    untouched = torch.ones(512 * 256, dtype=torch.bool)
    untouched[slots[slots >= 0].long()] = False
    assert not bool(kc.cpu().view(512 * 256, -1)[untouched].any()) and not bool(vc.cpu().view(512 * 256, -1)[untouched].any())
    assert int((slots >= 0).sum()) == case.n_valid


@pytest.mark.gpu
def test_stage_decode_inputs_copies_and_hands_over_tokens(dev):
    """The staging kernel copies the pinned buffer bit for bit and replaces exactly the input
    ids whose index names a row of the previous step's tokens (-1 and out-of-range keep the
    host's value)."""
    from nanovllm_amd import _lib
    lib = _lib.load()
    n, n_prev, nbytes = 37, 19, 4096
    ids_off, idx_off = 256, 1024                                    # int64 ids, int32 indices inside the buffer
    host = torch.randint(0, 255, (nbytes,), dtype=torch.uint8).pin_memory()
    ids = host[ids_off: ids_off + 8 * n].view(torch.int64)
    idx = host[idx_off: idx_off + 4 * n].view(torch.int32)
    g = torch.Generator().manual_seed(0)
    ids.copy_(torch.randint(0, 150000, (n,), generator=g))
    idx.copy_(torch.randint(-1, n_prev + 3, (n,), generator=g, dtype=torch.int32))   # includes -1 and too large
    prev = torch.randint(0, 150000, (n_prev,), generator=g).to(dev)
    dst = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    rc = lib.nva_stage_decode_inputs(dst.data_ptr(), host.data_ptr(), nbytes, ids_off, idx_off, n, prev.data_ptr(),
                                     n_prev, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = host.clone()
    want_ids = want[ids_off: ids_off + 8 * n].view(torch.int64)
    take = (idx >= 0) & (idx < n_prev)
    want_ids[take] = prev.cpu()[idx[take].long()]
    assert torch.equal(dst.cpu(), want)
    assert take.any() and (~take).any()
    # without previous tokens it is a plain copy
    rc = lib.nva_stage_decode_inputs(dst.data_ptr(), host.data_ptr(), nbytes, ids_off, idx_off, n, None, 0,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(dst.cpu(), host)
