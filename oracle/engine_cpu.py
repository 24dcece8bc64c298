"""CPU restatement of the reference's model step around the hot path.  TEST INFRASTRUCTURE.

Used by tests/ (end-to-end parity of the HIP path inside a Qwen3 stack) and by bench.py's
cpu_baseline leg (the reference semantics timed on the host cores).  Never imported by the
product package.

``forward`` follows nanovllm/models/qwen3.py (Qwen3Attention.forward :69-82,
Qwen3DecoderLayer.forward :140-153, Qwen3Model.forward :167-177, compute_logits via
nanovllm/layers/embed_head.py:56-61) on plain CPU tensors, with the four hot-path ops taken
from oracle.hotpath exactly where nanovllm/layers/attention.py:59-75 calls them.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from . import glue, hotpath


@dataclass
class StepContext:
    """The fields of nanovllm/utils/context.py:5-14, CPU tensors."""
    is_prefill: bool
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_k: Optional[torch.Tensor] = None
    slot_mapping: Optional[torch.Tensor] = None
    context_lens: Optional[torch.Tensor] = None
    block_tables: Optional[torch.Tensor] = None


def attention_forward(q, k, v, k_cache, v_cache, ctx: StepContext, scale: float, precision: str):
    """nanovllm/layers/attention.py:59-75 with the oracle ops."""
    if k_cache is not None and k_cache.numel():
        hotpath.store_kvcache(k, v, k_cache, v_cache, ctx.slot_mapping)
    if ctx.is_prefill:
        if ctx.block_tables is not None:
            o = hotpath.varlen_prefill_attention(q, None, None, ctx.cu_seqlens_q, ctx.cu_seqlens_k, scale,
                                                 k_cache, v_cache, ctx.block_tables, precision)
        else:
            o = hotpath.varlen_prefill_attention(q, k, v, ctx.cu_seqlens_q, ctx.cu_seqlens_k, scale,
                                                 precision=precision)
    else:
        o = hotpath.paged_decode_attention(q, k_cache, v_cache, ctx.context_lens, ctx.block_tables, scale, precision)
    return o.to(q.dtype)


def forward(weights: Dict[str, torch.Tensor], cfg, input_ids, positions, ctx: StepContext, kv_cache,
            rope_cache, precision: str = "sdpa"):
    """Hidden states after the final norm.  ``weights`` is the product model's state_dict on the
    CPU; ``kv_cache`` is ``[2, layers, blocks, 256, Hkv, Dh]`` or None (warm-up: no cache)."""
    hq, hkv, d, eps = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps
    hidden = F.embedding(input_ids, weights["embed_tokens"])
    residual = None
    for l in range(cfg.num_hidden_layers):
        w = lambda name: weights[f"layers.{l}.{name}"]
        if residual is None:
            residual, hidden = hidden, glue.rms_norm(hidden, w("input_layernorm"), eps)
        else:
            hidden, residual = glue.add_rms_norm(hidden, residual, w("input_layernorm"), eps)
        qkv = F.linear(hidden, w("qkv_proj"))
        q, k, v = glue.qk_norm_rope(qkv, positions, w("q_norm"), w("k_norm"), rope_cache, hq, hkv, d, eps)
        kc = kv_cache[0, l] if kv_cache is not None else None
        vc = kv_cache[1, l] if kv_cache is not None else None
        o = attention_forward(q, k, v, kc, vc, ctx, d ** -0.5, precision)
        hidden = F.linear(o.flatten(1, -1), w("o_proj"))
        hidden, residual = glue.add_rms_norm(hidden, residual, w("post_attention_layernorm"), eps)
        hidden = F.linear(glue.silu_and_mul(F.linear(hidden, w("gate_up_proj"))), w("down_proj"))
    hidden, _ = glue.add_rms_norm(hidden, residual, weights["norm"], eps)
    return hidden


def compute_logits(weights, cfg, hidden, ctx: StepContext):
    if ctx.is_prefill:
        hidden = hidden[(ctx.cu_seqlens_q[1:] - 1).long()].contiguous()
    head = weights["embed_tokens"] if cfg.tie_word_embeddings else weights["lm_head"]
    return F.linear(hidden, head)


def context_from_host_inputs(h: dict, is_prefill: bool) -> StepContext:
    """Build the step context from the dict the product's build_prefill_inputs /
    build_decode_inputs return (numpy arrays)."""
    t = lambda a, dt: None if a is None else torch.from_numpy(a).to(dt)
    if is_prefill:
        return StepContext(True, t(h["cu_seqlens_q"], torch.int32), t(h["cu_seqlens_k"], torch.int32),
                           t(h["slot_mapping"], torch.int32), None, t(h["block_tables"], torch.int32))
    return StepContext(False, slot_mapping=t(h["slot_mapping"], torch.int32),
                       context_lens=t(h["context_lens"], torch.int32), block_tables=t(h["block_tables"], torch.int32))


def random_weights(cfg, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16 weights ~ N(0, 0.02) with the product model's parameter names (norm weights are 1)."""
    g = torch.Generator().manual_seed(seed)
    h, d, i = cfg.hidden_size, cfg.head_dim, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * d, cfg.num_key_value_heads * d
    n = lambda *s: (torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16)
    ones = lambda s: torch.ones(s, dtype=torch.bfloat16)
    w = {"embed_tokens": n(cfg.vocab_size, h), "norm": ones(h)}
    if not cfg.tie_word_embeddings:
        w["lm_head"] = n(cfg.vocab_size, h)
    for l in range(cfg.num_hidden_layers):
        p = f"layers.{l}."
        w.update({p + "qkv_proj": n(q + 2 * kv, h), p + "o_proj": n(h, q), p + "gate_up_proj": n(2 * i, h),
                  p + "down_proj": n(h, i), p + "q_norm": ones(d), p + "k_norm": ones(d),
                  p + "input_layernorm": ones(h), p + "post_attention_layernorm": ones(h)})
    return w


def baseline(cfg, prompts: List[List[int]], params, num_requests: int = 16, max_new_tokens: int = 32,
             budget_s: float = 30.0) -> dict:
    """cpu_baseline for the end-to-end workload: the first ``num_requests`` requests of the bench
    mix, outputs capped at ``max_new_tokens``, run through the same scheduler / block manager
    with the CPU oracle as the device path.  Returns output tok/s on this host."""
    from nanovllm_amd.engine import EngineConfig, SamplingParams, Scheduler, Sequence
    from nanovllm_amd.engine.model_runner import build_decode_inputs, build_prefill_inputs

    weights = random_weights(cfg, 0)
    rope = glue.build_rope_cache(cfg.head_dim, 4096, cfg.rope_theta)
    ecfg = EngineConfig(cfg, max_model_len=4096, num_kvcache_blocks=64)
    kv = torch.zeros(2, cfg.num_hidden_layers, 64, 256, cfg.num_key_value_heads, cfg.head_dim, dtype=torch.bfloat16)
    sched = Scheduler(ecfg)
    total = 0
    for p, sp in list(zip(prompts, params))[:num_requests]:
        n = min(sp.max_tokens, max_new_tokens)
        total += n
        sched.add(Sequence(p, SamplingParams(temperature=sp.temperature, max_tokens=n, ignore_eos=True)))
    g = torch.Generator().manual_seed(0)
    t0 = time.perf_counter()
    done = 0
    with torch.inference_mode():
        while not sched.is_finished():
            seqs, is_prefill = sched.schedule()
            h = (build_prefill_inputs if is_prefill else build_decode_inputs)(seqs, 256)
            ctx = context_from_host_inputs(h, is_prefill)
            hidden = forward(weights, cfg, torch.from_numpy(h["input_ids"]), torch.from_numpy(h["positions"]), ctx,
                             kv, rope, "sdpa")
            logits = compute_logits(weights, cfg, hidden, ctx)
            temps = torch.tensor([s.temperature for s in seqs])
            noise = torch.empty(logits.shape, dtype=torch.float32).exponential_(1.0, generator=g)
            sched.postprocess(seqs, hotpath.sample(logits, temps, noise).tolist())
            done += len(seqs)
            if time.perf_counter() - t0 > budget_s:
                break
    dt = time.perf_counter() - t0
    return {"value": round(done / dt, 2), "unit": "tok/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{num_requests} requests ({done} of {total} output tokens generated in {dt:.1f} s, "
                      f"{sum(len(p) for p in prompts[:num_requests])} prompt tokens); same scheduler and block "
                      "manager, eager torch CPU ops (bf16 SDPA attention, index_copy scatter, eager sampler)",
            "seconds": round(dt, 2)}
