"""Element-wise / normalisation glue between the GEMMs of a Qwen3 layer, on the GPU.

Thin wrappers over the fused C-ABI kernels (csrc/glue.hip) that replace the reference's
torch.compile'd fusions: nanovllm/layers/layernorm.py:16-40, rotary_embedding.py:6-48 with
the per-head q/k norms of nanovllm/models/qwen3.py:76-79, and activation.py:11-14.
"""
from __future__ import annotations

import torch

from .. import _lib

_BF16 = torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``bf16(x * rsqrt(mean(x^2) + eps)) * weight`` over the last dim of a 2-D tensor."""
    assert x.dim() == 2 and x.dtype == _BF16 and x.stride(1) == 1 and x.is_cuda
    out = torch.empty((x.shape[0], x.shape[1]), dtype=_BF16, device=x.device)
    rc = _lib.load().nva_rms_norm(x.data_ptr(), x.stride(0), None, 0, weight.data_ptr(), out.data_ptr(), None,
                                  x.shape[0], x.shape[1], float(eps), _stream())
    _lib.check(rc, "nva_rms_norm")
    return out


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """Returns ``(normed(x + residual), bf16(x + residual))``."""
    assert x.dim() == 2 and x.dtype == _BF16 and x.stride(1) == 1 and x.is_cuda
    assert residual.shape == x.shape and residual.dtype == _BF16 and residual.stride(1) == 1
    out = torch.empty((x.shape[0], x.shape[1]), dtype=_BF16, device=x.device)
    res_out = torch.empty_like(out)
    rc = _lib.load().nva_rms_norm(x.data_ptr(), x.stride(0), residual.data_ptr(), residual.stride(0),
                                  weight.data_ptr(), out.data_ptr(), res_out.data_ptr(),
                                  x.shape[0], x.shape[1], float(eps), _stream())
    _lib.check(rc, "nva_rms_norm")
    return out, res_out


def gather_last_rms_norm(x: torch.Tensor, residual, cu_seqlens_q: torch.Tensor, weight: torch.Tensor,
                         eps: float) -> torch.Tensor:
    """Final (add +) RMSNorm of the last row of every sequence of a prefill batch: the rows
    ``x[cu_seqlens_q[1:] - 1]`` of nanovllm/layers/embed_head.py:58-60, normalised as
    nanovllm/models/qwen3.py:176 does for all rows -- without touching the others."""
    assert x.dim() == 2 and x.dtype == _BF16 and x.stride(1) == 1 and x.is_cuda
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.is_contiguous() and cu_seqlens_q.is_cuda
    batch = cu_seqlens_q.numel() - 1
    out = torch.empty((max(batch, 0), x.shape[1]), dtype=_BF16, device=x.device)
    if residual is not None:
        assert residual.shape == x.shape and residual.dtype == _BF16 and residual.stride(1) == 1
    rc = _lib.load().nva_gather_last_rms_norm(
        x.data_ptr(), x.stride(0), None if residual is None else residual.data_ptr(),
        0 if residual is None else residual.stride(0), cu_seqlens_q.data_ptr(), weight.data_ptr(),
        out.data_ptr(), batch, x.shape[0], x.shape[1], float(eps), _stream())
    _lib.check(rc, "nva_gather_last_rms_norm")
    return out


def build_rope_cache(head_dim: int, max_position: int, base: float, device) -> torch.Tensor:
    """``[max_position, head_dim]`` fp32: cos in the first half of a row, sin in the second
    (the table of nanovllm/layers/rotary_embedding.py:28-35)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float, device=device) / head_dim))
    t = torch.arange(max_position, dtype=torch.float, device=device)
    freqs = torch.outer(t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()


def qk_norm_rope(qkv: torch.Tensor, positions: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                 rope_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, eps: float,
                 kv_store=None):
    """Per-head RMSNorm of q and k, then the rotary embedding; optionally also the KV scatter.

    Returns ``(q, k, v)`` with q, k fresh contiguous ``[N, H, Dh]`` tensors and v a strided
    view into ``qkv`` -- the layouts nanovllm/models/qwen3.py:74-79 hands to the attention layer.
    ``kv_store=(k_cache, v_cache, slot_mapping)`` additionally writes the rotated key rows and
    the value rows to their cache slots in the same kernel (what ``store_kvcache`` would do
    next, nanovllm/layers/attention.py:62-63); the attention layer is then called with
    ``kv_stored=True``.
    """
    n = qkv.shape[0]
    assert qkv.dim() == 2 and qkv.dtype == _BF16 and qkv.stride(1) == 1 and qkv.is_cuda
    assert qkv.shape[1] == (num_heads + 2 * num_kv_heads) * head_dim
    assert positions.dtype == torch.int64 and positions.numel() == n and positions.is_contiguous()
    assert rope_cache.dtype == torch.float32 and rope_cache.is_contiguous() and rope_cache.shape[1] == head_dim
    q = torch.empty((n, num_heads, head_dim), dtype=_BF16, device=qkv.device)
    k = torch.empty((n, num_kv_heads, head_dim), dtype=_BF16, device=qkv.device)
    kc = vc = sm = None
    num_slots = 0
    if kv_store is not None:
        k_cache, v_cache, slot_mapping = kv_store
        d = num_kv_heads * head_dim
        assert k_cache.dtype == _BF16 and v_cache.dtype == _BF16 and k_cache.stride(1) == d and v_cache.stride(1) == d
        assert slot_mapping.dtype == torch.int32 and slot_mapping.numel() == n and slot_mapping.is_contiguous()
        kc, vc, sm, num_slots = k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(), k_cache.numel() // d
    rc = _lib.load().nva_qk_norm_rope(qkv.data_ptr(), qkv.stride(0), positions.data_ptr(), q_weight.data_ptr(),
                                      k_weight.data_ptr(), rope_cache.data_ptr(), rope_cache.shape[0],
                                      q.data_ptr(), k.data_ptr(), kc, vc, sm, num_slots,
                                      n, num_heads, num_kv_heads, head_dim, float(eps), _stream())
    _lib.check(rc, "nva_qk_norm_rope")
    v = qkv[:, (num_heads + num_kv_heads) * head_dim:].view(n, num_kv_heads, head_dim)
    return q, k, v


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    assert x.dim() == 2 and x.dtype == _BF16 and x.stride(1) == 1 and x.shape[1] % 2 == 0 and x.is_cuda
    inter = x.shape[1] // 2
    out = torch.empty((x.shape[0], inter), dtype=_BF16, device=x.device)
    rc = _lib.load().nva_silu_and_mul(x.data_ptr(), x.stride(0), out.data_ptr(), x.shape[0], inter, _stream())
    _lib.check(rc, "nva_silu_and_mul")
    return out
