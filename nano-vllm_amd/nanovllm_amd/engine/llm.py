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
        # Decode steps are launched one step ahead of their tokens: while the GPU runs step t the
        # host reads the tokens of step t-1, retires finished sequences and prepares step t+1.
        self.lookahead = config.decode_lookahead and not config.enforce_eager
        self._inflight = None                       # (DecodeHandle, token positions) not yet committed
        self.stats = {"prefill_steps": 0, "decode_steps": 0, "prefill_tokens": 0, "decode_tokens": 0,
                      "prefill_s": 0.0, "decode_s": 0.0}

    def add_request(self, prompt: Union[str, List[int]], sampling_params: SamplingParams) -> None:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("string prompts need a tokenizer; pass token ids instead")
            prompt = self.tokenizer.encode(prompt)
        self.scheduler.add(Sequence(prompt, sampling_params))

    def step(self):
        """One scheduling iteration.  Returns ``([(seq_id, completion ids) of finished requests],
        tokens processed: positive for prefill, negative for decode)`` like the reference's
        ``LLMEngine.step`` (llm_engine.py:48-54); with lookahead a request is reported when its
        last token has been read back, one iteration after the step that sampled it."""
        t0 = perf_counter()
        sch, runner = self.scheduler, self.model_runner
        finished = []
        # admission (prefix hashes, recompute of preempted sequences) needs every token in place
        if self._inflight is not None and (sch.waiting or not sch.running):
            finished += self._commit_inflight()
        if sch.is_finished():
            return self._report(finished), 0
        seqs, is_prefill = sch.schedule()
        if not is_prefill and self.lookahead and runner.can_launch_ahead(len(seqs)):
            handle = runner.launch_decode(seqs, self._inflight[0] if self._inflight else None)
            where = sch.advance(seqs)
            if self._inflight is not None:
                finished += self._commit_inflight()
            self._inflight = (handle, where)
        else:
            if self._inflight is not None:          # a decode batch beyond the captured sizes
                finished += self._commit_inflight()
            token_ids = runner.run(seqs, is_prefill)
            sch.postprocess(seqs, token_ids)
            finished += [s for s in seqs if s.is_finished]
        num_tokens = sum(len(s) for s in seqs) if is_prefill else -len(seqs)
        kind = "prefill" if is_prefill else "decode"
        self.stats[kind + "_steps"] += 1
        self.stats[kind + "_tokens"] += abs(num_tokens)
        self.stats[kind + "_s"] += perf_counter() - t0
        return self._report(finished), num_tokens

    def _commit_inflight(self):
        handle, where = self._inflight
        self._inflight = None
        return self.scheduler.commit(handle.seqs, where, handle.tokens())

    @staticmethod
    def _report(seqs):
        return [(s.seq_id, s.completion_token_ids) for s in seqs]

    def is_finished(self) -> bool:
        return self.scheduler.is_finished() and self._inflight is None

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
