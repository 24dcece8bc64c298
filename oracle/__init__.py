"""CPU oracle for the nano-vllm attention hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, as eager PyTorch ops on the CPU, the semantics of the four
device operations the reference runs on its hot path:

  * ``store_kvcache``                 nanovllm/layers/attention.py:10-40   (Triton)
  * paged single-query decode         nanovllm/layers/attention.py:71-74   (flash_attn_with_kvcache)
  * causal varlen prefill w/ prefix   nanovllm/layers/attention.py:59-70   (flash_attn_varlen_func)
  * temperature / exponential-race    nanovllm/layers/sampler.py:10-15     (torch.compile)

``flash-attn`` (version unpinned in the reference's pyproject.toml:18) is a third-party
CUDA wheel that is absent from the reference tree; its published semantics are restated
here: GQA mapping ``h_kv = h_q // (Hq // Hkv)``, paged layout ``[num_blocks, page, Hkv, Dh]``,
bottom-right aligned causal mask when ``seqlen_k > seqlen_q`` (flash-attn >= 2.1), fp32
softmax/accumulation and zero output for rows that see no keys.

For draws without a noise tensor the library's own scheme is restated as well: a tree of
inverse-CDF draws (``tree_draw``: row -> chunk of 8192 columns -> column group -> lane -> column), every level with its own Philox4x32-10 uniform (``philox4x32_10``, ``row_uniforms``; pinned
by the Random123 known-answer vectors), each level a walk through float64 running sums
(``inverse_cdf_bounds`` is the one-level form).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package, and only as the checker / the timed CPU baseline.  Nothing under the
product package imports it; the product fails loudly when its HIP library is missing.

Pin status (see tests/test_oracle_pins.py): every function below is checked against
independent float64 brute-force loops on tiny inputs, against library special cases
(``F.scaled_dot_product_attention`` on dense gathers) and against invariants.  The reference
ships no golden vectors, known-answer tests or fixtures for this path, so none are used.
"""
from .hotpath import (  # noqa: F401
    store_kvcache,
    gather_pages,
    paged_decode_attention,
    varlen_prefill_attention,
    philox4x32_10,
    row_uniforms,
    inverse_cdf_bounds,
    tree_draw,
    sample,
    sample_scores,
)
