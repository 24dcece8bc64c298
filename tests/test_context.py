"""The Context side channel keeps the reference's field names, defaults and call shape
(nanovllm/utils/context.py:5-27; nanovllm/engine/model_runner.py:160,178)."""
import dataclasses

import torch

import nanovllm_amd as nva


def test_context_fields_and_defaults():
    names = [f.name for f in dataclasses.fields(nva.Context)]
    # the reference's eight fields in its order (nanovllm/utils/context.py:7-15), then the one extension
    assert names == ["is_prefill", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k",
                     "slot_mapping", "context_lens", "block_tables", "decode_plan"]
    c = nva.Context()
    assert c.is_prefill is False and c.max_seqlen_q == 0 and c.max_seqlen_k == 0
    assert all(getattr(c, n) is None for n in names if n not in ("is_prefill", "max_seqlen_q", "max_seqlen_k"))


def test_set_get_reset_roundtrip():
    cq, ck, sm, bt = (torch.tensor([0, 3]), torch.tensor([0, 259]), torch.arange(3), torch.tensor([[1, 2]]))
    nva.set_context(True, cq, ck, 3, 259, sm, None, bt)            # eight positionals, prefill
    c = nva.get_context()
    assert c.is_prefill and c.cu_seqlens_q is cq and c.cu_seqlens_k is ck and c.max_seqlen_q == 3
    assert c.max_seqlen_k == 259 and c.slot_mapping is sm and c.context_lens is None and c.block_tables is bt
    nva.set_context(False, slot_mapping=sm, context_lens=ck, block_tables=bt)   # decode keywords
    d = nva.get_context()
    assert d is not c and not d.is_prefill and d.context_lens is ck and d.cu_seqlens_q is None
    nva.reset_context()
    assert nva.get_context() == nva.Context()


def test_attention_module_surface():
    a = nva.Attention(16, 128, 128 ** -0.5, 8)
    assert hasattr(a, "k_cache") and hasattr(a, "v_cache")         # how the runner discovers layers
    assert a.k_cache.numel() == 0 and a.v_cache.numel() == 0
    assert (a.num_heads, a.head_dim, a.num_kv_heads) == (16, 128, 8)
