"""Per-request sampling options (fields of nanovllm/sampling_params.py:5-8)."""
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False

    def __post_init__(self):
        # The reference forbids greedy decoding (temperature <= 1e-10).  Here temperature 0 is
        # accepted and means argmax; anything else must be a real temperature.
        assert self.temperature == 0 or self.temperature > 1e-10, "temperature must be 0 (greedy) or > 1e-10"
        assert self.max_tokens >= 1
