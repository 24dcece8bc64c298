"""CPU restatement of the element-wise steps either side of the attention hot path.
TEST INFRASTRUCTURE (same rules as the rest of oracle/).

Each function follows the reference line by line, including where it rounds to bf16:
  rms_norm / add_rms_norm   nanovllm/layers/layernorm.py:16-26 / :28-40
  apply_rope, qk_norm_rope  nanovllm/layers/rotary_embedding.py:6-15,37-48 and
                            nanovllm/models/qwen3.py:74-79
  silu_and_mul              nanovllm/layers/activation.py:11-14
  last_token_norm           nanovllm/models/qwen3.py:176 (final norm over all rows) followed by
                            nanovllm/layers/embed_head.py:58-60 (rows cu_seqlens_q[1:] - 1)
  build_rope_cache          nanovllm/layers/rotary_embedding.py:28-35 (cos | sin table)
"""
import torch
import torch.nn.functional as F


def rms_norm(x, weight, eps):
    orig = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return xf.to(orig) * weight


def add_rms_norm(x, residual, weight, eps):
    orig = x.dtype
    xf = x.float() + residual.float()
    new_residual = xf.to(orig)
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return xf.to(orig) * weight, new_residual


def last_token_norm(x, residual, cu_seqlens_q, weight, eps):
    """What the LM head receives in a prefill step: the final norm of every row, then the last
    row of every sequence (torch indexing: a negative index counts from the end)."""
    normed = rms_norm(x, weight, eps) if residual is None else add_rms_norm(x, residual, weight, eps)[0]
    last_indices = cu_seqlens_q[1:].long() - 1
    return normed[last_indices].contiguous()


def build_rope_cache(head_dim, max_position, base):
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    t = torch.arange(max_position, dtype=torch.float)
    freqs = torch.einsum("i,j -> ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def apply_rope(x, cos, sin):
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    y1 = x1 * cos - x2 * sin
    y2 = x2 * cos + x1 * sin
    return torch.cat((y1, y2), dim=-1).to(x.dtype)


def qk_norm_rope(qkv, positions, q_weight, k_weight, rope_cache, num_heads, num_kv_heads, head_dim, eps):
    n = qkv.shape[0]
    q_size, kv_size = num_heads * head_dim, num_kv_heads * head_dim
    q, k, v = qkv.split([q_size, kv_size, kv_size], dim=-1)
    q = rms_norm(q.reshape(n, num_heads, head_dim), q_weight, eps)
    k = rms_norm(k.reshape(n, num_kv_heads, head_dim), k_weight, eps)
    v = v.view(n, num_kv_heads, head_dim)
    cos, sin = rope_cache[positions].unsqueeze(1).chunk(2, dim=-1)
    return apply_rope(q, cos, sin), apply_rope(k, cos, sin), v


def silu_and_mul(x):
    gate, up = x.chunk(2, -1)
    return F.silu(gate) * up
