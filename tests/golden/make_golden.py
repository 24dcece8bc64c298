#!/usr/bin/env python3
"""Writes tests/golden/hotpath_small.npz: expected outputs of the CPU oracle on small seeded cases.

The reference ships no golden vectors for this path and cannot be imported in this environment
(it needs the CUDA-only flash-attn wheel), so these vectors come from this repository's own
oracle (oracle/hotpath.py), whose functions are pinned independently in tests/test_oracle_pins.py.
They freeze the oracle's results so that later edits to it, or to the input generators, cannot go
unnoticed.  Inputs are NOT stored: they are rebuilt from seeds by nanovllm_amd.synthetic and
checked against the SHA-256 digests stored here.

    python tests/golden/make_golden.py          # rewrites hotpath_small.npz
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "nano-vllm_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import oracle  # noqa: E402
from helpers import digest  # noqa: E402
from nanovllm_amd import synthetic  # noqa: E402


def cases():
    """name -> (inputs digest, dict of expected arrays); the same builders are used by the tests."""
    out = {}
    sc = synthetic.scatter_case(seed=11, n_tokens=200, num_kv_heads=2, num_blocks=3, skip_fraction=0.1)
    kc, vc = sc.k_cache.clone(), sc.v_cache.clone()
    oracle.store_kvcache(sc.key, sc.value, kc, vc, sc.slot_mapping)
    out["scatter"] = (digest(sc.key, sc.value, sc.slot_mapping),
                      {"k_cache_digest": np.frombuffer(bytes.fromhex(digest(kc)), dtype=np.uint8),
                       "v_cache_digest": np.frombuffer(bytes.fromhex(digest(vc)), dtype=np.uint8),
                       "slot_of_token_0": np.array([int(sc.slot_mapping[0])]),
                       "k_row_token_0": sc.key[0].reshape(-1).view(torch.int16).numpy()})
    dc = synthetic.decode_case(seed=12, num_heads=4, num_kv_heads=2, num_blocks=14,
                               context_lens=[1, 255, 256, 257, 700, 0, 33])
    out["decode"] = (digest(dc.q, dc.k_cache, dc.v_cache, dc.context_lens, dc.block_tables),
                     {"out": oracle.paged_decode_attention(dc.q, dc.k_cache, dc.v_cache, dc.context_lens,
                                                           dc.block_tables, dc.scale, "fp32").numpy()})
    pc = synthetic.prefill_case(seed=13, num_heads=2, num_kv_heads=1, q_lens=[40, 130, 7, 64],
                                prefix_blocks=[1, 0, 2, 0], num_blocks=10)
    ek, ev = pc.k_cache.clone(), pc.v_cache.clone()
    oracle.store_kvcache(pc.k, pc.v, ek, ev, pc.slot_mapping)
    out["prefill"] = (digest(pc.q, pc.k, pc.v, pc.k_cache, pc.v_cache, pc.cu_seqlens_q, pc.cu_seqlens_k,
                             pc.slot_mapping, pc.block_tables),
                      {"out": oracle.varlen_prefill_attention(pc.q, None, None, pc.cu_seqlens_q, pc.cu_seqlens_k,
                                                              pc.scale, ek, ev, pc.block_tables, "fp32").numpy()})
    sm = synthetic.sampler_case(seed=14, batch=12, vocab=5003, temperature=0.7)
    scores = oracle.sample_scores(sm.logits, sm.temperatures, sm.noise)
    top2 = scores.topk(2, dim=-1)
    out["sampler"] = (digest(sm.logits, sm.temperatures, sm.noise),
                      {"tokens": oracle.sample(sm.logits, sm.temperatures, sm.noise).numpy(),
                       "top2_scores": top2.values.numpy(), "top2_index": top2.indices.numpy()})
    return out


def main():
    flat = {}
    for name, (dig, arrays) in cases().items():
        flat[f"{name}/inputs_sha256"] = np.frombuffer(bytes.fromhex(dig), dtype=np.uint8)
        for k, v in arrays.items():
            flat[f"{name}/{k}"] = v
    path = os.path.join(HERE, "hotpath_small.npz")
    np.savez_compressed(path, **flat)
    print("wrote", path, os.path.getsize(path), "bytes", "torch", torch.__version__)


if __name__ == "__main__":
    main()
