"""``LLM(...).generate(prompts, sampling_params)`` -- the reference's user API on one GPU.

Same call shape and return value as nanovllm/engine/llm_engine.py:59-93 (a list of
``{"text", "token_ids"}`` in request order).  Prompts are lists of token ids; strings need a
tokenizer directory, which is optional because no tokenizer files exist offline.
"""
from __future__ import annotations

import dataclasses
from time import perf_counter
from typing import List, Union

from .config import EngineConfig, ModelConfig
from .model_runner import ModelRunner
from .sampling_params import SamplingParams
from .scheduler import Scheduler
from .sequence import Sequence


class LLMEngine:

    def __init__(self, model: Union[ModelConfig, str], tokenizer=None, **kwargs):
        known = {f.name for f in dataclasses.fields(EngineConfig)}
        config = EngineConfig(model, **{k: v for k, v in kwargs.items() if k in known})
        self.config = config
        self.tokenizer = tokenizer
        if tokenizer is not None and getattr(tokenizer, "eos_token_id", None) is not None:
            config.eos = tokenizer.eos_token_id
        self.model_runner = ModelRunner(config)
        self.scheduler = Scheduler(config)
        self.stats = {"prefill_steps": 0, "decode_steps": 0, "prefill_tokens": 0, "decode_tokens": 0,
                      "prefill_s": 0.0, "decode_s": 0.0}

    def add_request(self, prompt: Union[str, List[int]], sampling_params: SamplingParams) -> None:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("string prompts need a tokenizer; pass token ids instead")
            prompt = self.tokenizer.encode(prompt)
        self.scheduler.add(Sequence(prompt, sampling_params))

    def step(self):
        t0 = perf_counter()
        seqs, is_prefill = self.scheduler.schedule()
        token_ids = self.model_runner.run(seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        outputs = [(s.seq_id, s.completion_token_ids) for s in seqs if s.is_finished]
        num_tokens = sum(len(s) for s in seqs) if is_prefill else -len(seqs)
        kind = "prefill" if is_prefill else "decode"
        self.stats[kind + "_steps"] += 1
        self.stats[kind + "_tokens"] += abs(num_tokens)
        self.stats[kind + "_s"] += perf_counter() - t0
        return outputs, num_tokens

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    def generate(self, prompts, sampling_params, use_tqdm: bool = False):
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        for prompt, sp in zip(prompts, sampling_params):
            self.add_request(prompt, sp)
        done = {}
        while not self.is_finished():
            finished, _ = self.step()
            for seq_id, toks in finished:
                done[seq_id] = toks
        decode = (lambda t: self.tokenizer.decode(t)) if self.tokenizer is not None else (lambda t: "")
        return [{"text": decode(done[i]), "token_ids": done[i]} for i in sorted(done)]


class LLM(LLMEngine):
    pass
