"""Shared helpers for the parity tests."""
import hashlib

import torch

MAX_ABS = 2e-2    # attention tolerance against the fp32-accumulated oracle, bf16 inputs/outputs
MEAN_ABS = 2e-3


def assert_attn_close(got_bf16, want_fp32, what=""):
    got = got_bf16.detach().float().cpu().reshape(-1)
    want = want_fp32.detach().float().cpu().reshape(-1)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    diff = (got - want).abs()
    mx, mean = float(diff.max()) if diff.numel() else 0.0, float(diff.mean()) if diff.numel() else 0.0
    assert mx <= MAX_ABS and mean <= MEAN_ABS, f"{what}: max-abs {mx:.4g} mean-abs {mean:.4g}"
    return mx, mean


def bits(t):
    """bf16 tensor -> int16 view for bit-exact comparison."""
    return t.detach().cpu().contiguous().view(torch.int16)


def digest(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        t = t.detach().cpu().contiguous()
        if t.dtype == torch.bfloat16:
            t = t.view(torch.int16)
        h.update(t.numpy().tobytes())
    return h.hexdigest()


def assert_sampled_like_oracle(tokens, scores, rel=2e-5):
    """tokens [B] from the device; scores [B, V] = oracle's p / E.  The device token must be
    the oracle's argmax, or a column whose oracle score ties the maximum to fp32 rounding."""
    tokens = tokens.detach().cpu()
    best = scores.argmax(-1)
    top = scores.gather(1, best[:, None])[:, 0]
    mine = scores.gather(1, tokens[:, None])[:, 0]
    exact = tokens == best
    near = mine >= top * (1 - rel)
    assert bool((exact | near).all()), f"rows differ beyond fp32 ties: {(~(exact | near)).nonzero().flatten().tolist()}"
    return int((~exact).sum())
