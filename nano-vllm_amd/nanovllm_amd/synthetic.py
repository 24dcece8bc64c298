"""Seeded synthetic inputs for the hot-path kernels (CPU tensors; callers move them).

The shapes are the ones the kernels meet inside nano-vllm:
  scatter  -- ``store_kvcache(key, value, k_cache, v_cache, slot_mapping)``
              (nanovllm/layers/attention.py:33-40)
  decode   -- ``context_lens`` / ``block_tables`` as ``prepare_decode`` builds them
              (nanovllm/engine/model_runner.py:162-179): tables padded with -1
  prefill  -- ``cu_seqlens_q/k``, ``slot_mapping`` and ``block_tables`` as ``prepare_prefill``
              builds them (model_runner.py:126-160) when some sequences hit the prefix cache
  sampler  -- bf16 logits ``[B, vocab]``, fp32 temperatures, fp32 Exp(1) noise
Everything is drawn from ``torch.Generator`` objects seeded by the caller, so the same
inputs can be rebuilt on the GPU box without shipping data files.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

BLOCK_SIZE = 256  # nanovllm/config.py:17,22 and nanovllm/engine/sequence.py:15


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def _randn_bf16(shape, g):
    return torch.randn(shape, generator=g, dtype=torch.float32).to(torch.bfloat16)


@dataclass
class ScatterCase:
    key: torch.Tensor
    value: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    slot_mapping: torch.Tensor
    n_valid: int

    @property
    def algorithmic_bytes(self) -> int:
        d = self.key.shape[1] * self.key.shape[2]
        # read + write of one K row and one V row per stored token, plus the slot ids
        return self.n_valid * (2 * d * 2) * 2 + self.slot_mapping.numel() * 4


def scatter_case(seed=0, n_tokens=4096, num_kv_heads=8, head_dim=128, num_blocks=512,
                 skip_fraction=0.05, strided_value=False, block_size=BLOCK_SIZE) -> ScatterCase:
    """KV-cache slot scatter: distinct slots from a permutation, a fraction set to -1.

    ``strided_value`` makes ``value`` a view into a wider buffer, as in the model where v is
    a slice of the fused qkv projection (nanovllm/models/qwen3.py:74-78).
    """
    g = _gen(seed)
    num_slots = num_blocks * block_size
    key = _randn_bf16((n_tokens, num_kv_heads, head_dim), g)
    if strided_value:
        wide = _randn_bf16((n_tokens, 4 * num_kv_heads * head_dim), g)
        value = wide[:, 3 * num_kv_heads * head_dim:].view(n_tokens, num_kv_heads, head_dim)
    else:
        value = _randn_bf16((n_tokens, num_kv_heads, head_dim), g)
    slots = torch.randperm(num_slots, generator=g)[:n_tokens].to(torch.int32)
    n_skip = int(round(n_tokens * skip_fraction))
    if n_skip:
        skip = torch.randperm(n_tokens, generator=g)[:n_skip]
        slots[skip] = -1
    k_cache = torch.zeros(num_blocks, block_size, num_kv_heads, head_dim, dtype=torch.bfloat16)
    v_cache = torch.zeros_like(k_cache)
    return ScatterCase(key, value, k_cache, v_cache, slots, n_tokens - n_skip)


@dataclass
class DecodeCase:
    q: torch.Tensor               # [B, Hq, Dh] bf16
    k_cache: torch.Tensor         # [num_blocks, block, Hkv, Dh] bf16
    v_cache: torch.Tensor
    context_lens: torch.Tensor    # [B] int32
    block_tables: torch.Tensor    # [B, max_blocks] int32, -1 padded
    scale: float

    @property
    def algorithmic_bytes(self) -> int:
        hkv, dh = self.k_cache.shape[2], self.k_cache.shape[3]
        kv = int(self.context_lens.to(torch.int64).sum()) * hkv * dh * 2 * 2
        return kv + 2 * self.q.numel() * 2


def decode_tables(context_lens, num_blocks, g, block_size=BLOCK_SIZE, width=None):
    """Per-sequence block ids drawn without replacement from the pool, -1 padded."""
    need = [(int(c) + block_size - 1) // block_size for c in context_lens]
    total = sum(need)
    assert total <= num_blocks, "pool too small for the drawn context lengths"
    perm = torch.randperm(num_blocks, generator=g)[:total].to(torch.int32)
    width = max(need + [1]) if width is None else width
    tables = torch.full((len(need), width), -1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(need):
        tables[i, :n] = perm[at:at + n]
        at += n
    return tables


def decode_case(seed=0, batch=64, num_heads=16, num_kv_heads=8, head_dim=128, num_blocks=1024,
                ctx_lo=100, ctx_hi=2048, block_size=BLOCK_SIZE, cache=None,
                context_lens=None) -> DecodeCase:
    """Paged decode attention inputs.  ``cache=(k_cache, v_cache)`` reuses an existing pool."""
    g = _gen(seed)
    if context_lens is None:
        context_lens = torch.randint(ctx_lo, ctx_hi + 1, (batch,), generator=g, dtype=torch.int32)
    else:
        context_lens = torch.as_tensor(context_lens, dtype=torch.int32)
        batch = context_lens.numel()
    tables = decode_tables(context_lens.tolist(), num_blocks, g, block_size)
    q = _randn_bf16((batch, num_heads, head_dim), g)
    if cache is None:
        k_cache = _randn_bf16((num_blocks, block_size, num_kv_heads, head_dim), g)
        v_cache = _randn_bf16((num_blocks, block_size, num_kv_heads, head_dim), g)
    else:
        k_cache, v_cache = cache
    return DecodeCase(q, k_cache, v_cache, context_lens, tables, head_dim ** -0.5)


@dataclass
class PrefillCase:
    q: torch.Tensor               # [total_q, Hq, Dh]
    k: torch.Tensor               # [total_q, Hkv, Dh]  new keys (to be scattered)
    v: torch.Tensor
    k_cache: torch.Tensor         # prefix blocks already populated
    v_cache: torch.Tensor
    cu_seqlens_q: torch.Tensor    # [B+1] int32
    cu_seqlens_k: torch.Tensor
    max_seqlen_q: int
    max_seqlen_k: int
    slot_mapping: torch.Tensor    # [total_q] int32
    block_tables: Optional[torch.Tensor]   # [B, max_blocks] int32 or None (no prefix anywhere)
    scale: float
    prefix_lens: list = field(default_factory=list)

    @property
    def algorithmic_flops(self) -> int:
        hq, dh = self.q.shape[1], self.q.shape[2]
        lq = (self.cu_seqlens_q[1:] - self.cu_seqlens_q[:-1]).to(torch.int64)
        lk = (self.cu_seqlens_k[1:] - self.cu_seqlens_k[:-1]).to(torch.int64)
        pairs = int((lq * (lk - lq) + lq * (lq + 1) // 2).sum())
        return 4 * dh * hq * pairs


def prefill_case(seed=0, batch=16, num_heads=16, num_kv_heads=8, head_dim=128, num_blocks=128,
                 q_lo=100, q_hi=1024, prefix_fraction=0.5, max_prefix_blocks=3,
                 block_size=BLOCK_SIZE, q_lens=None, prefix_blocks=None) -> PrefillCase:
    """Causal varlen prefill where a fraction of the sequences own cached prefix blocks.

    Sequence ``b`` has ``prefix_b`` (a multiple of ``block_size``) tokens already in the cache
    and ``Lq_b`` new tokens: ``cu_seqlens_q`` runs over ``Lq``, ``cu_seqlens_k`` over
    ``prefix + Lq``, ``slot_mapping`` places new token ``t`` at
    ``block_table[(prefix+t) // bs] * bs + (prefix+t) % bs``, and ``block_tables`` is present
    iff any prefix is non-empty (model_runner.py:153-154).
    """
    g = _gen(seed)
    if q_lens is None:
        q_lens = torch.randint(q_lo, q_hi + 1, (batch,), generator=g).tolist()
    batch = len(q_lens)
    if prefix_blocks is None:
        n_pref = int(round(batch * prefix_fraction))
        has = torch.zeros(batch, dtype=torch.bool)
        has[torch.randperm(batch, generator=g)[:n_pref]] = True
        draw = torch.randint(1, max_prefix_blocks + 1, (batch,), generator=g)
        prefix_blocks = [int(d) if h else 0 for d, h in zip(draw.tolist(), has.tolist())]
    prefix_lens = [p * block_size for p in prefix_blocks]
    k_lens = [p + l for p, l in zip(prefix_lens, q_lens)]
    tables = decode_tables(k_lens, num_blocks, g, block_size)
    total_q = sum(q_lens)
    q = _randn_bf16((total_q, num_heads, head_dim), g)
    k = _randn_bf16((total_q, num_kv_heads, head_dim), g)
    v = _randn_bf16((total_q, num_kv_heads, head_dim), g)
    k_cache = torch.zeros(num_blocks, block_size, num_kv_heads, head_dim, dtype=torch.bfloat16)
    v_cache = torch.zeros_like(k_cache)
    slots = torch.empty(total_q, dtype=torch.int32)
    at = 0
    for b in range(batch):
        for j in range(prefix_blocks[b]):            # cached prefix content
            blk = int(tables[b, j])
            k_cache[blk] = _randn_bf16((block_size, num_kv_heads, head_dim), g)
            v_cache[blk] = _randn_bf16((block_size, num_kv_heads, head_dim), g)
        pos = torch.arange(prefix_lens[b], k_lens[b])
        slots[at:at + q_lens[b]] = (tables[b, pos // block_size].to(torch.int64) * block_size
                                    + pos % block_size).to(torch.int32)
        at += q_lens[b]
    cu_q = torch.tensor([0] + q_lens, dtype=torch.int64).cumsum(0).to(torch.int32)
    cu_k = torch.tensor([0] + k_lens, dtype=torch.int64).cumsum(0).to(torch.int32)
    any_prefix = any(prefix_blocks)
    return PrefillCase(q, k, v, k_cache, v_cache, cu_q, cu_k, max(q_lens), max(k_lens), slots,
                       tables if any_prefix else None, head_dim ** -0.5, prefix_lens)


@dataclass
class SamplerCase:
    logits: torch.Tensor          # [B, V] bf16
    temperatures: torch.Tensor    # [B] fp32
    noise: torch.Tensor           # [B, V] fp32 Exp(1)

    @property
    def algorithmic_bytes(self) -> int:
        return self.logits.numel() * 2 + self.noise.numel() * 4


def sampler_case(seed=0, batch=64, vocab=151936, temperature=0.6, logit_scale=2.0) -> SamplerCase:
    g = _gen(seed)
    logits = (torch.randn((batch, vocab), generator=g) * logit_scale).to(torch.bfloat16)
    temps = torch.full((batch,), float(temperature), dtype=torch.float32)
    noise = torch.empty((batch, vocab), dtype=torch.float32).exponential_(1.0, generator=g)
    return SamplerCase(logits, temps, noise)
