"""Pins for oracle/glue.py (RMSNorm, rotary embedding, SwiGLU gate): closed forms and
invariants that do not share code with the restatement."""
import math

import torch

from oracle import glue


def test_rms_norm_closed_forms():
    x = torch.full((3, 64), 2.0, dtype=torch.bfloat16)
    w = torch.linspace(0.5, 1.5, 64).to(torch.bfloat16)
    out = glue.rms_norm(x, w, 0.0)                       # constant row: x / |x| = 1 -> out = w
    assert torch.equal(out, w.expand(3, 64))
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 128, generator=g).to(torch.bfloat16)
    ones = torch.ones(128, dtype=torch.bfloat16)
    y = glue.rms_norm(x, ones, 1e-6).double()
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5, dtype=torch.float64), atol=2e-2)   # unit RMS
    ref = (x.double() / x.double().pow(2).mean(-1, keepdim=True).add(1e-6).sqrt())
    assert (y - ref).abs().max() < 2e-2
    # scale invariance (eps = 0): norm(4x) == norm(x) exactly, powers of two are exact in bf16
    assert torch.equal(glue.rms_norm(x * 4, ones, 0.0), glue.rms_norm(x, ones, 0.0))


def test_add_rms_norm_is_norm_of_the_sum_and_returns_rounded_sum():
    g = torch.Generator().manual_seed(1)
    x, r = torch.randn(4, 256, generator=g).to(torch.bfloat16), torch.randn(4, 256, generator=g).to(torch.bfloat16)
    w = torch.randn(256, generator=g).to(torch.bfloat16)
    out, res = glue.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(res, (x.float() + r.float()).to(torch.bfloat16))
    s = x.double() + r.double()
    ref = s / s.pow(2).mean(-1, keepdim=True).add(1e-6).sqrt() * w.double()
    assert (out.double() - ref).abs().max() < 5e-2
    # zero residual: same as the plain norm
    assert torch.equal(glue.add_rms_norm(x, torch.zeros_like(x), w, 1e-6)[0], glue.rms_norm(x, w, 1e-6))


def test_last_token_norm_rows_by_float64_loop():
    """Row b of the result is the norm of input row cu[b+1]-1, computed here element by element in
    float64 without the restatement's code; an empty span repeats the previous row, index -1 wraps."""
    g = torch.Generator().manual_seed(4)
    x, r = torch.randn(9, 64, generator=g).to(torch.bfloat16), torch.randn(9, 64, generator=g).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(64, generator=g)).to(torch.bfloat16)
    cu = torch.tensor([0, 0, 3, 3, 8, 9], dtype=torch.int32)          # spans: empty (wraps to row 8), 3, empty, 5, 1
    out = glue.last_token_norm(x, r, cu, w, 1e-6)
    assert out.shape == (5, 64)
    for b, src in enumerate([8, 2, 2, 7, 8]):
        s = [float(x[src, i]) + float(r[src, i]) for i in range(64)]
        inv = 1.0 / math.sqrt(sum(v * v for v in s) / 64 + 1e-6)
        for i in range(64):
            want = s[i] * inv * float(w[i])
            assert abs(float(out[b, i]) - want) <= 2.0 ** -6 * max(abs(want), 1e-3), (b, i)
    # without a residual the plain norm of the same rows
    assert torch.equal(glue.last_token_norm(x, None, cu, w, 1e-6), glue.rms_norm(x, w, 1e-6)[[8, 2, 2, 7, 8]])


def test_rope_table_and_rotation_properties():
    cache = glue.build_rope_cache(128, 64, 1e6)
    assert cache.shape == (64, 128)
    assert torch.allclose(cache[0, :64], torch.ones(64)) and torch.allclose(cache[0, 64:], torch.zeros(64))
    for p, i in [(1, 0), (7, 3), (63, 63)]:              # angle = p * base^(-2i/d)
        ang = p * 1e6 ** (-2 * i / 128)
        assert abs(float(cache[p, i]) - math.cos(ang)) < 1e-5 and abs(float(cache[p, 64 + i]) - math.sin(ang)) < 1e-5
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 2, 128, generator=g)
    pos = torch.tensor([0, 1, 5, 9, 20, 63])
    cos, sin = cache[pos].unsqueeze(1).chunk(2, -1)
    y = glue.apply_rope(x, cos, sin)
    assert torch.equal(y[0], x[0])                                             # position 0: identity
    assert torch.allclose(y.pow(2).sum(-1), x.pow(2).sum(-1), rtol=1e-5)       # rotations keep the norm
    # pairs (i, i+64) rotate together: element i of y depends only on x[i], x[i+64]
    x2 = x.clone()
    x2[..., 3] += 1.0
    d = (glue.apply_rope(x2, cos, sin) - y).abs().sum(dim=(0, 1))
    assert set(d.nonzero().flatten().tolist()) <= {3, 67}
    # relative-position property: <rope(q, p1), rope(k, p2)> depends on p1 - p2 only
    q, k = torch.randn(1, 1, 128, generator=g), torch.randn(1, 1, 128, generator=g)

    def dot(p1, p2):
        c1, s1 = cache[p1:p1 + 1].unsqueeze(1).chunk(2, -1)
        c2, s2 = cache[p2:p2 + 1].unsqueeze(1).chunk(2, -1)
        return float((glue.apply_rope(q, c1, s1) * glue.apply_rope(k, c2, s2)).sum())
    assert abs(dot(10, 3) - dot(40, 33)) < 1e-3 and abs(dot(10, 3) - dot(10, 4)) > 1e-4


def test_qk_norm_rope_layouts():
    g = torch.Generator().manual_seed(3)
    n, hq, hkv, d = 5, 4, 2, 128
    qkv = torch.randn(n, (hq + 2 * hkv) * d, generator=g).to(torch.bfloat16)
    cache = glue.build_rope_cache(d, 32, 1e6)
    pos = torch.tensor([0, 3, 3, 31, 7])
    ones = torch.ones(d, dtype=torch.bfloat16)
    q, k, v = glue.qk_norm_rope(qkv, pos, ones, ones, cache, hq, hkv, d, 1e-6)
    assert q.shape == (n, hq, d) and k.shape == (n, hkv, d) and v.shape == (n, hkv, d)
    assert torch.equal(v.reshape(n, -1), qkv[:, (hq + hkv) * d:])              # values untouched
    # position 0: no rotation, just the per-head norm
    assert torch.equal(q[0], glue.rms_norm(qkv[0, : hq * d].view(hq, d), ones, 1e-6))
    # tokens 1 and 2 share a position: swapping their rows swaps the outputs
    qkv2 = qkv.clone()
    qkv2[[1, 2]] = qkv[[2, 1]]
    q2, k2, _ = glue.qk_norm_rope(qkv2, pos, ones, ones, cache, hq, hkv, d, 1e-6)
    assert torch.equal(q2[1], q[2]) and torch.equal(k2[2], k[1])


def test_silu_and_mul_known_values():
    x = torch.tensor([[0.0, 1.0, -1.0, 20.0, 2.0, 3.0, 4.0, 0.5]], dtype=torch.bfloat16)
    out = glue.silu_and_mul(x).float()
    want = [0.0 * 2.0, 1 / (1 + math.exp(-1)) * 3.0, -1 / (1 + math.exp(1)) * 4.0, 20.0 * 0.5]
    assert out.shape == (1, 4)
    assert all(abs(float(o) - w) <= 8e-3 * max(1.0, abs(w)) for o, w in zip(out[0], want))
