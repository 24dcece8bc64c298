"""Attention layer and its three device ops, backed by the gfx950 C-ABI library.

Drop-in for nanovllm/layers/attention.py: ``Attention(num_heads, head_dim, scale,
num_kv_heads)`` with ``k_cache`` / ``v_cache`` attributes (the runner finds attention layers
by those two attributes, nanovllm/engine/model_runner.py:113-117) and
``forward(q, k, v) -> o`` driven by the global Context.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import _lib
from .context import DecodePlan, get_context

BLOCK_SIZE = 256
_BF16 = torch.bfloat16
_PLAN_BUILD, _PLAN_REUSE = 0, 1          # NVA_PLAN_BUILD / NVA_PLAN_REUSE of the C header


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("nanovllm_amd ops run on the GPU only (there is no CPU fallback)")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """Scatter the rows of ``key``/``value`` into the paged caches at ``slot_mapping``.

    Same signature and the same four layout checks as the reference's ``store_kvcache``
    (nanovllm/layers/attention.py:33-40).  A slot of -1 skips its row.
    """
    n, num_kv_heads, head_dim = key.shape
    d = num_kv_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == d and v_cache.stride(1) == d
    assert slot_mapping.numel() == n
    if n == 0:
        return
    assert key.dtype == _BF16 and value.dtype == _BF16 and k_cache.dtype == _BF16 and v_cache.dtype == _BF16
    assert slot_mapping.dtype == torch.int32 and slot_mapping.is_contiguous()
    _need_cuda(key, value, k_cache, v_cache, slot_mapping)
    num_slots = k_cache.numel() // d
    lib = _lib.load()
    rc = lib.nva_store_kvcache(key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0),
                               k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                               n, num_kv_heads, head_dim, num_slots, _stream())
    _lib.check(rc, "nva_store_kvcache")


_workspaces: dict = {}
_retired_workspaces: list = []
_last_builder: dict = {}                 # device -> the DecodePlan (or None) of the last call that derived a work split there


def _decode_workspace(device, nbytes: int) -> torch.Tensor:
    """Scratch for the decode kernel's split partials.

    One buffer per device, shared by every layer (calls are ordered on one stream).  It
    only grows outside graph capture: a captured graph
    must be preceded by an eager warm-up call of the same shape, which is what the runner
    does before capturing each batch size (nanovllm/engine/model_runner.py:232-234).
    A buffer that is replaced by a larger one is kept alive until the process ends: graphs
    captured earlier (and the work split they reuse) hold its address.
    """
    ws = _workspaces.get(device)
    if ws is None or ws.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("decode workspace must be allocated by an eager warm-up call before graph capture")
        if ws is not None:
            _retired_workspaces.append(ws)
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[device] = ws
    return ws


def paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           context_lens: torch.Tensor, block_tables: torch.Tensor, scale: float,
                           out: Optional[torch.Tensor] = None, plan: Optional[DecodePlan] = None) -> torch.Tensor:
    """One query token per sequence against its paged keys/values.

    ``q`` is ``[B, Hq, Dh]`` or ``[B, 1, Hq, Dh]``; the result has the shape of the
    reference's ``flash_attn_with_kvcache`` output, ``[B, 1, Hq, Dh]``
    (nanovllm/layers/attention.py:72-74).  Calls that pass the same ``plan`` promise the same
    ``context_lens``/``block_tables`` contents and run in order on one stream: the first
    derives the work split, the others reuse it.
    """
    if q.dim() == 4:
        assert q.shape[1] == 1
        q = q.squeeze(1)
    b, hq, dh = q.shape
    num_blocks, block_size, hkv, dh2 = k_cache.shape
    assert dh2 == dh and v_cache.shape == k_cache.shape
    assert q.dtype == _BF16 and k_cache.dtype == _BF16 and v_cache.dtype == _BF16
    assert q.stride(-1) == 1 and q.stride(1) == dh
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert context_lens.dtype == torch.int32 and context_lens.numel() == b and context_lens.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] == b
    assert block_tables.stride(1) == 1
    _need_cuda(q, k_cache, v_cache, context_lens, block_tables)
    if out is None:
        out = torch.empty((b, 1, hq, dh), dtype=_BF16, device=q.device)
    else:
        assert out.is_contiguous() and out.numel() == b * hq * dh and out.dtype == _BF16
    if b == 0:
        return out
    max_blocks = block_tables.shape[1]
    lib = _lib.load()
    nbytes = lib.nva_paged_decode_workspace_bytes(b, hq, dh, max(max_blocks, 1))
    ws = _decode_workspace(q.device, nbytes)
    mode = _PLAN_BUILD
    if plan is not None:
        key = (ws.data_ptr(), b, hq, hkv, num_blocks, block_tables.data_ptr(), context_lens.data_ptr())
        if plan.key is None:
            plan.key = key
        elif plan.key != key:
            raise ValueError("decode plan reused with a different batch, geometry, table or workspace")
        elif _last_builder.get(q.device) is plan:
            mode = _PLAN_REUSE
        # else: another decode call derived its own split in the shared workspace since this plan's
        # first call and overwrote the stored one -- derive it again
    if mode == _PLAN_BUILD:
        _last_builder[q.device] = plan
    rc = lib.nva_paged_decode_attn_planned(q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                           block_tables.data_ptr(), block_tables.stride(0), max_blocks,
                                           context_lens.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(),
                                           b, hq, hkv, dh, block_size, num_blocks, float(scale), mode, _stream())
    _lib.check(rc, "nva_paged_decode_attn_planned")
    return out


def varlen_prefill_attention(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                             cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                             max_seqlen_q: int, max_seqlen_k: int, scale: float,
                             block_table: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal packed attention; the keyword set of the reference's ``flash_attn_varlen_func``
    call (nanovllm/layers/attention.py:67-70).  With ``block_table`` given, ``k``/``v`` are
    the paged caches ``[num_blocks, 256, Hkv, Dh]``; otherwise packed ``[total_k, Hkv, Dh]``.
    """
    total_q, hq, dh = q.shape
    assert q.dtype == _BF16 and q.stride(-1) == 1 and q.stride(1) == dh
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert cu_seqlens_q.is_contiguous() and cu_seqlens_k.is_contiguous()
    batch = cu_seqlens_q.numel() - 1
    assert cu_seqlens_k.numel() == batch + 1
    _need_cuda(q, k, v, cu_seqlens_q, cu_seqlens_k, block_table)
    out = torch.empty((total_q, hq, dh), dtype=_BF16, device=q.device)
    if total_q == 0 or batch <= 0:
        return out
    lib = _lib.load()
    if block_table is not None:
        num_blocks, block_size, hkv, dh2 = k.shape
        assert dh2 == dh and v.shape == k.shape and k.is_contiguous() and v.is_contiguous()
        assert k.dtype == _BF16 and v.dtype == _BF16
        assert block_table.dtype == torch.int32 and block_table.shape[0] == batch and block_table.stride(1) == 1
        rc = lib.nva_varlen_prefill_attn(q.data_ptr(), q.stride(0), None, 0, None, 0,
                                         k.data_ptr(), v.data_ptr(), block_table.data_ptr(),
                                         block_table.stride(0), block_table.shape[1],
                                         cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), batch,
                                         int(max_seqlen_q), int(max_seqlen_k), out.data_ptr(),
                                         hq, hkv, dh, block_size, num_blocks, float(scale), _stream())
    else:
        total_k, hkv, dh2 = k.shape
        assert dh2 == dh and v.shape == k.shape and k.dtype == _BF16 and v.dtype == _BF16
        assert k.stride(-1) == 1 and v.stride(-1) == 1 and k.stride(1) == dh and v.stride(1) == dh
        rc = lib.nva_varlen_prefill_attn(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0),
                                         v.data_ptr(), v.stride(0), None, None, None, 0, 0,
                                         cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), batch,
                                         int(max_seqlen_q), int(max_seqlen_k), out.data_ptr(),
                                         hq, hkv, dh, BLOCK_SIZE, 0, float(scale), _stream())
    _lib.check(rc, "nva_varlen_prefill_attn")
    return out


def _decode_plan_of(ctx) -> Optional[DecodePlan]:
    """The work-split plan the layers of this forward pass share: the one on the context, made here by
    the first layer if the runner did not provide any.  Eager runs and graph captures never share one."""
    capturing = torch.cuda.is_current_stream_capturing()
    plan = getattr(ctx, "decode_plan", None)
    if plan is None or plan.capturing != capturing:
        plan = DecodePlan(capturing)
        try:
            ctx.decode_plan = plan
        except AttributeError:                     # a foreign context object without room for it: no sharing
            return None
    return plan


class Attention(nn.Module):
    """Paged-KV attention layer: scatter the new K/V rows, then prefill or decode attention.

    Mirrors nanovllm/layers/attention.py:43-75.  ``k_cache``/``v_cache`` start as empty
    tensors and are replaced by ``[num_blocks, 256, Hkv, Dh]`` views by the runner.
    """

    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kv_stored: bool = False) -> torch.Tensor:
        """``kv_stored=True`` says the caller already wrote this step's K/V rows to the cache
        (the fused norm + rope + scatter kernel does); the default keeps the reference's
        behaviour of scattering here."""
        ctx = get_context()
        k_cache, v_cache = self.k_cache, self.v_cache
        have_cache = k_cache.numel() > 0 and v_cache.numel() > 0
        if have_cache and not kv_stored:
            store_kvcache(k, v, k_cache, v_cache, ctx.slot_mapping)
        if ctx.is_prefill:
            paged = ctx.block_tables is not None       # some sequence reads cached prefix blocks
            return varlen_prefill_attention(
                q, k_cache if paged else k, v_cache if paged else v,
                ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.max_seqlen_q, ctx.max_seqlen_k,
                self.scale, block_table=ctx.block_tables)
        return paged_decode_attention(q, k_cache, v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                                      plan=_decode_plan_of(ctx))
