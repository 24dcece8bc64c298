"""Qwen3 decoder stack for one GPU (architecture of nanovllm/models/qwen3.py).

qkv / gate-up projections are stored fused, the LM head is tied to the embedding when the
config says so, and every attention layer is a ``nanovllm_amd.Attention`` whose
``k_cache`` / ``v_cache`` the runner fills in.  Weights are random (normal, std 0.02):
no checkpoint is available offline and throughput does not depend on the values.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from ..attention import Attention
from ..context import get_context
from . import layers
from .config import ModelConfig


class DecoderLayer(nn.Module):

    def __init__(self, cfg: ModelConfig, rope_cache: torch.Tensor):
        super().__init__()
        h, d = cfg.hidden_size, cfg.head_dim
        self.num_heads, self.num_kv_heads, self.head_dim, self.eps = cfg.num_attention_heads, cfg.num_key_value_heads, d, cfg.rms_norm_eps
        q_size, kv_size = self.num_heads * d, self.num_kv_heads * d
        self.qkv_proj = nn.Parameter(torch.empty(q_size + 2 * kv_size, h))
        self.o_proj = nn.Parameter(torch.empty(h, q_size))
        self.gate_up_proj = nn.Parameter(torch.empty(2 * cfg.intermediate_size, h))
        self.down_proj = nn.Parameter(torch.empty(h, cfg.intermediate_size))
        self.q_norm = nn.Parameter(torch.ones(d))
        self.k_norm = nn.Parameter(torch.ones(d))
        self.input_layernorm = nn.Parameter(torch.ones(h))
        self.post_attention_layernorm = nn.Parameter(torch.ones(h))
        self.rope_cache = rope_cache                     # shared, not a parameter
        self.attn = Attention(self.num_heads, d, d ** -0.5, self.num_kv_heads)

    def forward(self, positions, hidden, residual):
        if residual is None:
            residual, hidden = hidden, layers.rms_norm(hidden, self.input_layernorm, self.eps)
        else:
            hidden, residual = layers.add_rms_norm(hidden, residual, self.input_layernorm, self.eps)
        qkv = F.linear(hidden, self.qkv_proj)
        attn = self.attn
        fused_store = attn.k_cache.numel() > 0                 # no cache yet during the warm-up pass
        q, k, v = layers.qk_norm_rope(qkv, positions, self.q_norm, self.k_norm, self.rope_cache,
                                      self.num_heads, self.num_kv_heads, self.head_dim, self.eps,
                                      kv_store=(attn.k_cache, attn.v_cache, get_context().slot_mapping)
                                      if fused_store else None)
        o = attn(q, k, v, kv_stored=fused_store)
        hidden = F.linear(o.flatten(1, -1), self.o_proj)
        hidden, residual = layers.add_rms_norm(hidden, residual, self.post_attention_layernorm, self.eps)
        hidden = F.linear(layers.silu_and_mul(F.linear(hidden, self.gate_up_proj)), self.down_proj)
        return hidden, residual


class Qwen3ForCausalLM(nn.Module):

    def __init__(self, cfg: ModelConfig, max_position: int, device, seed: int = 0):
        super().__init__()
        self.cfg = cfg
        rope = layers.build_rope_cache(cfg.head_dim, max_position, cfg.rope_theta, device)
        self.embed_tokens = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden_size))
        self.layers = nn.ModuleList([DecoderLayer(cfg, rope) for _ in range(cfg.num_hidden_layers)])
        self.norm = nn.Parameter(torch.ones(cfg.hidden_size))
        self.lm_head = self.embed_tokens if cfg.tie_word_embeddings else nn.Parameter(
            torch.empty(cfg.vocab_size, cfg.hidden_size))
        gen = torch.Generator(device=device).manual_seed(seed)
        with torch.no_grad():
            for p in self.parameters():
                if p.dim() == 2:
                    p.normal_(0.0, 0.02, generator=gen)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        hidden, residual = self.forward_layers(input_ids, positions, None, None, 0, len(self.layers))
        return self.finish(hidden, residual)

    def forward_layers(self, input_ids, positions, hidden, residual, first: int, last: int):
        """Layers ``[first, last)``; the embedding lookup is part of the slice that starts at 0.
        Lets the runner capture the stack as several consecutive graphs."""
        if first == 0:
            hidden, residual = F.embedding(input_ids, self.embed_tokens), None
        for layer in self.layers[first:last]:
            hidden, residual = layer(positions, hidden, residual)
        return hidden, residual

    def finish(self, hidden, residual) -> torch.Tensor:
        hidden, _ = layers.add_rms_norm(hidden, residual, self.norm, self.cfg.rms_norm_eps)
        return hidden

    def prefill_logits(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """``compute_logits(forward(...))`` of a prefill step with the final norm applied to the
        rows the LM head reads only: the last token of every sequence
        (nanovllm/models/qwen3.py:176, nanovllm/layers/embed_head.py:56-61)."""
        hidden, residual = self.forward_layers(input_ids, positions, None, None, 0, len(self.layers))
        rows = layers.gather_last_rms_norm(hidden, residual, get_context().cu_seqlens_q, self.norm,
                                           self.cfg.rms_norm_eps)
        return F.linear(rows, self.lm_head)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """Logits of the last token of every sequence (nanovllm/layers/embed_head.py:56-61)."""
        ctx = get_context()
        if ctx.is_prefill:
            last = ctx.cu_seqlens_q[1:] - 1
            hidden = hidden[last.long()].contiguous()
        return F.linear(hidden, self.lm_head)
