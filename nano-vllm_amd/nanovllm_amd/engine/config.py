"""Engine and model configuration (own dataclasses; no transformers config object).

EngineConfig keeps the field names and defaults of nanovllm/config.py:7-18.  ModelConfig
carries the architecture numbers a Qwen3 ``config.json`` would (the reference reads them
through transformers.AutoConfig, nanovllm/config.py:24).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Optional


@dataclass
class ModelConfig:
    vocab_size: int = 151936
    hidden_size: int = 1024
    num_hidden_layers: int = 28
    num_attention_heads: int = 16
    num_key_value_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 3072
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    max_position_embeddings: int = 40960
    tie_word_embeddings: bool = True
    name: str = "qwen3"

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        with open(path) as f:
            raw = json.load(f)
        keys = {f_.name for f_ in cls.__dataclass_fields__.values()}
        cfg = cls(**{k: v for k, v in raw.items() if k in keys})
        if "head_dim" not in raw:
            cfg.head_dim = cfg.hidden_size // cfg.num_attention_heads
        return cfg

    def param_count(self) -> int:
        h, i, v, l = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers
        q, kv = self.num_attention_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        per_layer = h * (q + 2 * kv) + q * h + 3 * h * i + 2 * h + 2 * self.head_dim
        return l * per_layer + v * h * (1 if self.tie_word_embeddings else 2) + h


def qwen3_0_6b() -> ModelConfig:
    """Qwen3-0.6B architecture: 28 layers, hidden 1024, 16/8 heads of 128, MLP 3072."""
    return ModelConfig(name="qwen3-0.6b")


def qwen3_8b() -> ModelConfig:
    """Qwen3-8B architecture: 36 layers, hidden 4096, 32/8 heads of 128, MLP 12288."""
    return ModelConfig(hidden_size=4096, num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8,
                       intermediate_size=12288, tie_word_embeddings=False, name="qwen3-8b")


@dataclass
class EngineConfig:
    model: object = field(default_factory=qwen3_0_6b)     # ModelConfig, or a directory holding config.json
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    enforce_eager: bool = False
    hf_config: Optional[ModelConfig] = None
    eos: int = -1
    kvcache_block_size: int = 256
    num_kvcache_blocks: int = -1
    seed: int = 0
    decode_lookahead: bool = True                        # launch decode steps one step ahead of their tokens
    graph_bucket_step: int = 16                          # decode graphs are captured for batch sizes 1, 2, 4, 8 and every multiple of this

    def __post_init__(self):
        if isinstance(self.model, ModelConfig):
            self.hf_config = self.model
        else:
            assert os.path.isdir(self.model), f"{self.model} is not a directory"
            self.hf_config = ModelConfig.from_json(os.path.join(self.model, "config.json"))
        assert self.kvcache_block_size % 256 == 0
        assert self.kvcache_block_size == 256, "this engine keeps Sequence.block_size = 256 like nanovllm/engine/sequence.py:15 (the kernels take 256 * 2^k)"
        assert self.tensor_parallel_size == 1, "this build runs on one GPU"
        assert self.graph_bucket_step >= 1
        self.max_model_len = min(self.max_model_len, self.hf_config.max_position_embeddings)
        assert self.max_num_batched_tokens >= self.max_model_len
