"""MI355X-native attention hot path for nano-vllm (gfx950 HIP kernels behind a C ABI).

Public surface mirrors the reference modules it replaces:
  Attention, store_kvcache          nanovllm/layers/attention.py
  Sampler                           nanovllm/layers/sampler.py
  Context, get/set/reset_context    nanovllm/utils/context.py
"""
from .context import Context, get_context, set_context, reset_context  # noqa: F401
from .attention import Attention, store_kvcache, paged_decode_attention, varlen_prefill_attention  # noqa: F401
from .sampler import Sampler, sample  # noqa: F401
from . import _lib  # noqa: F401

__version__ = "0.1"
