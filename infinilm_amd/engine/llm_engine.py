"""The engine loop: schedule -> step function -> sample -> update, after the reference's
`LLMEngine.step` (python/infinilm/llm/llm.py:143-176) and `_update_requests` (:178-277)."""
from __future__ import annotations

import itertools
import time
from typing import Dict, List, Optional, Sequence

import torch

from ..sampling import Sampler, SamplingParams
from .request import FinishReason, InferenceRequest, RequestStatus
from .scheduler import Scheduler, SchedulerOutput
from .step import StepEntry, StepRunner


class LLMEngine:
    def __init__(self, runner: StepRunner, max_num_seqs: int, max_num_batched_tokens: int,
                 chunk_size: Optional[int] = None, policy: str = "optimistic", seed: int = 0,
                 eos_token_ids: Optional[Sequence[int]] = None, tokenizer=None):
        self.runner = runner
        self.model = runner.model
        spec = self.model.spec
        self.scheduler = Scheduler(runner.cache, max_num_seqs, max_num_batched_tokens, chunk_size, policy,
                                   max_positions=spec.max_positions)
        self.sampler = Sampler(seed)
        self.eos_token_ids = list(eos_token_ids if eos_token_ids is not None else spec.eos_token_ids)
        self.tokenizer = tokenizer
        self._ids = itertools.count()
        self.requests: Dict[str, InferenceRequest] = {}
        self.counters = {"steps": 0, "prompt_tokens": 0, "generated_tokens": 0, "schedule_s": 0.0, "step_s": 0.0,
                         "sample_s": 0.0, "update_s": 0.0}

    def add_request(self, prompt_token_ids: Sequence[int], sampling_params: Optional[SamplingParams] = None,
                    request_id: Optional[str] = None, prompt: Optional[str] = None) -> InferenceRequest:
        n = next(self._ids)
        rid = request_id if request_id is not None else f"req-{n}"
        if rid in self.requests and not self.requests[rid].is_finished():
            raise ValueError(f"request id {rid!r} is in use")
        V = self.model.spec.vocab_size
        for t in prompt_token_ids:
            if not 0 <= int(t) < V:
                raise ValueError(f"prompt token id {t} is outside the vocabulary of {V}")
        req = InferenceRequest(rid, [int(t) for t in prompt_token_ids], sampling_params or SamplingParams(), prompt,
                               self.eos_token_ids, key=n)
        self.requests[rid] = req
        self.scheduler.add_request(req)
        return req

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    def step(self) -> List[InferenceRequest]:
        """One step of the step function for whatever the scheduler picks; returns the requests
        that finished in it."""
        t0 = time.perf_counter()
        out = self.scheduler.schedule()
        t1 = time.perf_counter()
        self.counters["schedule_s"] += t1 - t0
        if not out.entries:
            if self.scheduler.waiting and not self.scheduler.running:
                req = self.scheduler.waiting.popleft()
                self.scheduler._fail(req, "no_capacity: the request cannot be admitted into an empty engine")
                return [req]
            return []
        entries = []
        for e in out.entries:
            toks = e.request.token_slice(e.start, e.num_tokens)
            entries.append(StepEntry(e.request.request_id, toks, [e.num_tokens - 1] if e.samples else []))
        logits = self.runner.step(entries)
        t2 = time.perf_counter()
        samplers = [(e.request.sampling_params, e.request.key, e.request.get_num_generated_tokens())
                    for e in out.entries if e.samples]
        tokens = self.sampler.sample(logits, samplers)   # brings the tokens to the host: waits for the step
        t3 = time.perf_counter()
        sampled = {e.request.request_id: t for e, t in zip((e for e in out.entries if e.samples), tokens)}
        done = self.scheduler.update(out, sampled)
        c = self.counters
        c["steps"] += 1
        if not out.decode_only:
            c["prompt_tokens"] += sum(e.num_tokens for e in out.entries if e.start < e.request.get_prompt_length())
        c["generated_tokens"] += len(tokens)
        c["step_s"] += t2 - t1
        c["sample_s"] += t3 - t2
        c["update_s"] += time.perf_counter() - t3
        if self.tokenizer is not None:
            for e in out.entries:
                if e.samples:
                    self._detokenize(e.request)
        return done

    def stats(self) -> dict:
        """Counters of the loop (steps, tokens run, host seconds spent scheduling, launching the step,
        sampling including the wait for the device, updating) and the scheduler's view of the cache
        (python/infinilm/llm/scheduler.py:579-598 for the latter)."""
        out = dict(self.counters)
        out["cache"] = self.scheduler.get_cache_stats()
        return out

    def _detokenize(self, req: InferenceRequest) -> None:
        text = self.tokenizer.decode(req.output_token_ids, skip_special_tokens=True)
        if text.endswith("�") and not req.is_finished():
            return  # an incomplete multi-byte character: hold back (python/infinilm/llm/llm.py:230-262)
        req.generated_text = text
        sp = req.sampling_params
        if not sp.ignore_eos and not req.is_finished():
            for s in sp.stop:
                if s and req.generated_text.endswith(s):
                    req.generated_text = req.generated_text[:-len(s)]
                    self.scheduler.abort(req)
                    req.status = RequestStatus.FINISHED
                    req.finish_reason = FinishReason.STOP_STRING
                    break

    def run_until_done(self) -> None:
        while self.has_unfinished():
            self.step()
