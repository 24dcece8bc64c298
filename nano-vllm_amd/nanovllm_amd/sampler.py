"""Token sampler backed by the fused gfx950 kernels.

Drop-in for nanovllm/layers/sampler.py: ``Sampler()(logits, temperatures) -> int64 [B]``, a
categorical draw from ``softmax(logits / T)``.  Given a tensor of ``E ~ Exp(1)`` draws the kernels
evaluate the reference's exponential race ``argmax(p / E)`` (replayable); without one -- what the
module interface does -- they draw from the same distribution by a tree of inverse-CDF steps with
Philox uniforms of 32 bits per level (conditional probabilities below 2**-32 are not resolved;
the reference's fp32 race has a comparable floor).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import _lib


STATIC_MAX_RECORDS = 131072          # NVA_SAMPLE_STATIC_MAX_RECORDS of the C header


def sample(logits: torch.Tensor, temperatures: torch.Tensor, noise: Optional[torch.Tensor] = None,
           seed: int = 0, offset: int = 0, static_scratch: bool = False) -> torch.Tensor:
    """``argmax(softmax(logits.float() / T) / clamp_min(E, 1e-10))`` per row.

    ``noise`` (fp32 ``[B, V]``) supplies ``E`` explicitly so a draw can be replayed; with
    ``noise=None`` the kernel draws the token from the same categorical distribution by a tree of
    inverse-CDF steps (chunk of 8192 columns, wavefront group, lane, column) with Philox uniforms
    keyed by ``(seed, offset)``.  Rows with temperature 0 return ``argmax(logits)``.
    ``static_scratch=True`` keeps the per-chunk records in the library's built-in device array
    (``nva_sample_static``: no workspace is allocated; calls on one GPU must not overlap) whenever
    the problem fits it, and falls back to a workspace tensor when it does not.
    """
    assert logits.dim() == 2 and logits.dtype == torch.bfloat16 and logits.stride(1) == 1
    b, vocab = logits.shape
    assert temperatures.dtype == torch.float32 and temperatures.numel() == b and temperatures.is_contiguous()
    if not logits.is_cuda:
        raise RuntimeError("nanovllm_amd ops run on the GPU only (there is no CPU fallback)")
    out = torch.empty(b, dtype=torch.int64, device=logits.device)
    if b == 0:
        return out
    if noise is not None:
        assert noise.dtype == torch.float32 and noise.shape == logits.shape and noise.stride(1) == 1
        assert noise.is_cuda
    lib = _lib.load()
    nptr, nstride = (None, 0) if noise is None else (noise.data_ptr(), noise.stride(0))
    if static_scratch and b * ((vocab + 2047) // 2048) <= STATIC_MAX_RECORDS:
        rc = lib.nva_sample_static(logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), nptr, nstride,
                                   int(seed) & 0xFFFFFFFFFFFFFFFF, int(offset) & 0xFFFFFFFFFFFFFFFF,
                                   out.data_ptr(), b, vocab, torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "nva_sample_static")
        return out
    nbytes = lib.nva_sample_workspace_bytes(b, vocab)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=logits.device)
    rc = lib.nva_sample(logits.data_ptr(), logits.stride(0), temperatures.data_ptr(),
                        None if noise is None else noise.data_ptr(),
                        0 if noise is None else noise.stride(0),
                        int(seed) & 0xFFFFFFFFFFFFFFFF, int(offset) & 0xFFFFFFFFFFFFFFFF,
                        out.data_ptr(), ws.data_ptr(), ws.numel(), b, vocab,
                        torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "nva_sample")
    return out


class Sampler(nn.Module):
    """``forward(logits, temperatures)`` as in nanovllm/layers/sampler.py:10-15.

    Each call advances a Philox offset, so successive calls draw afresh while a run
    with the same ``seed`` is reproducible.  The chunk records go to the library's built-in
    scratch array (a module's calls are ordered on one stream), so a step allocates only its
    output tokens.
    """

    def __init__(self, seed: int = 0, static_scratch: bool = True):
        super().__init__()
        self.seed = seed
        self.calls = 0
        self.static_scratch = static_scratch

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor) -> torch.Tensor:
        self.calls += 1
        return sample(logits, temperatures, None, self.seed, self.calls, self.static_scratch)
