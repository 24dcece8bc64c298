"""Minimal single-GPU serving harness around the hot-path kernels.

It exists so the kernels can be measured where they live -- inside a Qwen3-architecture
decoder driven by nano-vllm's scheduler / paged block manager / graph-replay loop
(reference: nanovllm/engine/*.py, nanovllm/models/qwen3.py).  Dense GEMMs, norms and the
MLP stay on PyTorch-ROCm; attention, KV scatter and sampling go through the C-ABI library.
"""
from .config import ModelConfig, EngineConfig, qwen3_0_6b, qwen3_8b  # noqa: F401
from .sampling_params import SamplingParams  # noqa: F401
from .sequence import Sequence, SequenceStatus  # noqa: F401
from .block_manager import BlockManager  # noqa: F401
from .scheduler import Scheduler  # noqa: F401
