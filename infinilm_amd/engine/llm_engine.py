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


class _Flight:
    """A step that has been launched: its plan, the sampled tokens on the device and on their way
    into pinned host memory.  `ahead_of`: 1 if it was launched before the step before it was booked."""
    __slots__ = ("out", "tokens_dev", "tokens_host", "arrived", "ahead_of")

    def __init__(self, out: SchedulerOutput):
        self.out = out
        self.tokens_dev = None
        self.tokens_host = None
        self.arrived = None
        self.ahead_of = 0

    def wait(self) -> List[int]:
        if self.tokens_host is None:
            return []
        self.arrived.synchronize()
        return self.tokens_host.tolist()


class LLMEngine:
    def __init__(self, runner: StepRunner, max_num_seqs: int, max_num_batched_tokens: int,
                 chunk_size: Optional[int] = None, policy: str = "optimistic", seed: int = 0,
                 eos_token_ids: Optional[Sequence[int]] = None, tokenizer=None, look_ahead: Optional[bool] = None):
        self.runner = runner
        # decode steps launched one ahead of the host's books: needs the recorded decode steps
        self.look_ahead = runner.enable_graph if look_ahead is None else bool(look_ahead) and runner.enable_graph
        self._flight: Optional[_Flight] = None
        self.model = runner.model
        spec = self.model.spec
        self.scheduler = Scheduler(runner.cache, max_num_seqs, max_num_batched_tokens, chunk_size, policy,
                                   max_positions=spec.max_positions)
        self.sampler = Sampler(seed)
        self.eos_token_ids = list(eos_token_ids if eos_token_ids is not None else spec.eos_token_ids)
        self.tokenizer = tokenizer
        self._ids = itertools.count()
        self.requests: Dict[str, InferenceRequest] = {}
        self.counters = {"steps": 0, "ahead_steps": 0, "prompt_tokens": 0, "generated_tokens": 0, "schedule_s": 0.0, "step_s": 0.0,
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

    # ---- one step ---------------------------------------------------------------------------------
    def _launch(self, out: SchedulerOutput) -> "_Flight":
        """Runs the scheduler's plan through the step function and the sampler; nothing waits for
        the device: the tokens are on their way into pinned host memory."""
        entries = []
        for e in out.entries:
            toks = e.request.token_slice(e.start, e.num_tokens)
            entries.append(StepEntry(e.request.request_id, toks, [e.num_tokens - 1] if e.samples else []))
        logits = self.runner.step(entries)
        rows = [(e.request.sampling_params, e.request.key, e.request.get_num_generated_tokens())
                for e in out.entries if e.samples]
        return self._sample(out, logits, rows)

    def _sample(self, out: SchedulerOutput, logits: torch.Tensor, rows) -> "_Flight":
        f = _Flight(out)
        if rows:
            f.tokens_dev = self.sampler.sample_device(logits, rows)
            f.tokens_host = torch.empty((len(rows),), dtype=torch.int32, pin_memory=True)
            f.tokens_host.copy_(f.tokens_dev, non_blocking=True)
            f.arrived = torch.cuda.Event()
            f.arrived.record()
        return f

    def _launch_ahead(self, flight: "_Flight") -> Optional["_Flight"]:
        """The decode step after `flight`, launched before `flight`'s tokens are back: its input tokens
        go from the sampler's output to the step on the device.  Only where the next step is known
        without them: `flight` holds one decoded token of every running request, nobody waits to be
        admitted, no request reaches its length with the token on its way, and the step function has
        the step prepared.  A request that ends for another reason (an end-of-sequence token, a stop
        string) has run one step in vain, which is never read."""
        sch = self.scheduler
        out = flight.out
        if not (self.look_ahead and out.decode_only and flight.tokens_dev is not None):
            return None
        if len(out.entries) != len(sch.running) or (sch.waiting and len(sch.running) < sch.max_num_seqs):
            return None
        for e in out.entries:
            req = e.request
            if req.is_finished():
                return None
            generated = req.get_num_generated_tokens() + 1      # once flight's token is in: the only one not booked
            if generated >= req.sampling_params.max_tokens or req.get_prompt_length() + generated >= sch.max_positions:
                return None
        ids = [e.request.request_id for e in out.entries]
        if not self.runner.ahead_ready(ids):
            return None
        nxt = SchedulerOutput(decode_only=True)
        nxt.entries = [type(e)(e.request, e.start + 1, 1, True) for e in out.entries]
        logits = self.runner.step_ahead(ids, flight.tokens_dev)
        rows = [(e.request.sampling_params, e.request.key, e.request.get_num_generated_tokens() + 1)
                for e in out.entries]
        f = self._sample(nxt, logits, rows)
        f.ahead_of = 1
        self.counters["ahead_steps"] += 1
        sch.log.append({"decode": len(ids), "portions": [], "preempted": 0,
                        "free_pages": [g.pool.num_free for g in sch.cache.groups]})
        return f

    def step(self) -> List[InferenceRequest]:
        """One step of the step function for whatever the scheduler picks; returns the requests
        that finished in it.  With `look_ahead`, the decode step after it is already launched when
        this one's tokens are waited for, so the device does not stand still while the host books."""
        t0 = time.perf_counter()
        flight, self._flight = self._flight, None
        if flight is not None and all(e.request.is_finished() for e in flight.out.entries):
            flight = None        # launched ahead for requests that have all ended since
        c = self.counters
        if flight is None:
            out = self.scheduler.schedule()
            t1 = time.perf_counter()
            c["schedule_s"] += t1 - t0
            if not out.entries:
                if self.scheduler.waiting and not self.scheduler.running:
                    req = self.scheduler.waiting.popleft()
                    self.scheduler._fail(req, "no_capacity: the request cannot be admitted into an empty engine")
                    return [req]
                return []
            flight = self._launch(out)
        else:
            t1 = t0
        ahead = self._launch_ahead(flight)
        t2 = time.perf_counter()
        out = flight.out
        tokens = flight.wait()           # brings the tokens to the host: waits for the step
        t3 = time.perf_counter()
        if flight.ahead_of:
            # launched before the step before it was booked: requests that ended with that one are left out
            live = [(e, t) for e, t in zip(out.entries, tokens) if not e.request.is_finished()]
            out.entries = [e for e, _ in live]
            tokens = [t for _, t in live]
        sampled = {e.request.request_id: t for e, t in zip((e for e in out.entries if e.samples), tokens)}
        done = self.scheduler.update(out, sampled)
        if ahead is not None:
            self.runner.commit_ahead([(e.request.request_id, sampled[e.request.request_id]) for e in out.entries
                                      if not e.request.is_finished()])
            self._flight = ahead
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
