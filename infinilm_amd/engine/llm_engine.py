"""The engine loop: schedule -> step function -> sample -> update, after the reference's
`LLMEngine.step` (python/infinilm/llm/llm.py:143-176) and `_update_requests` (:178-277)."""
from __future__ import annotations

import itertools
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
        out = self.scheduler.schedule()
        if not out.entries:
            if self.scheduler.waiting and not self.scheduler.running:
                req = self.scheduler.waiting.popleft()
                self.scheduler._fail(req, "no_capacity: the request cannot be admitted into an empty engine")
                return [req]
            return []
        entries = []
        for e in out.entries:
            toks = e.request.all_token_ids()[e.start:e.start + e.num_tokens]
            entries.append(StepEntry(e.request.request_id, toks, [e.num_tokens - 1] if e.samples else []))
        logits = self.runner.step(entries)
        samplers = [(e.request.sampling_params, e.request.key, e.request.get_num_generated_tokens())
                    for e in out.entries if e.samples]
        tokens = self.sampler.sample(logits, samplers)
        sampled = {e.request.request_id: t for e, t in zip((e for e in out.entries if e.samples), tokens)}
        done = self.scheduler.update(out, sampled)
        if self.tokenizer is not None:
            for e in out.entries:
                if e.samples:
                    self._detokenize(e.request)
        return done

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
