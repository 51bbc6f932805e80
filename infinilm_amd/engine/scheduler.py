"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees, and decides what happens when pages run out.

Reference: python/infinilm/llm/scheduler.py: FIFO waiting and running queues (:75-76), admission
with a token budget (:111-127) and a worst-case page check (:453-495), head-of-line blocking
(:202-215), a step is either all prompts or all decodes (:295-366), finishing frees pages
(:404-451).  The reference never cuts a prompt and never preempts: running out of pages in a
decode raises (python/infinilm/llm/cache_manager.py:321-324).

Here every step holds the running requests' decode tokens first, then portions of prompts (those
already begun, then new admissions) until the token budget or the batch size is used up.  Two
admission policies:
  reserve_full  the reference's check: a request enters only if the pages for its prompt and
                its max_tokens, plus what every running request may still need, fit the pool;
                pages then never run out.
  optimistic    a request enters if its first portion fits now.  When a later token finds no page,
                the most recently admitted running request is preempted: its pages go back, it
                returns to the front of the waiting queue and is recomputed (prompt and generated
                tokens) when it is admitted again.  A request that cannot fit the pool alone fails
                with FinishReason.ERROR when it is added.
The scheduler never touches the GPU: it plans against the cache manager's page counts.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional

from ..cache import CacheManager
from .request import FinishReason, InferenceRequest, RequestStatus


@dataclass
class ScheduledEntry:
    request: InferenceRequest
    start: int            # index of the first token of the portion in request.all_token_ids()
    num_tokens: int
    samples: bool         # the portion ends at the last known token: a new token is sampled from it


@dataclass
class SchedulerOutput:
    entries: List[ScheduledEntry] = field(default_factory=list)
    preempted: List[InferenceRequest] = field(default_factory=list)
    decode_only: bool = False    # known to hold nothing but decoded tokens (no token of a prompt)

    @property
    def num_tokens(self) -> int:
        return sum(e.num_tokens for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int,
                 chunk_size: Optional[int] = None, policy: str = "optimistic", max_positions: int = 1 << 30):
        if policy not in ("optimistic", "reserve_full"):
            raise ValueError(f"unknown admission policy {policy!r}")
        if max_num_seqs <= 0 or max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        self.cache = cache
        self.max_num_seqs = int(max_num_seqs)
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.chunk_size = int(chunk_size or max_num_batched_tokens)
        self.policy = policy
        self.max_positions = int(max_positions)
        self.waiting: Deque[InferenceRequest] = deque()
        self.running: List[InferenceRequest] = []
        self.finished: List[InferenceRequest] = []
        self._admissions = 0
        self.num_preemptions = 0
        self.log: Deque[Dict] = deque(maxlen=4096)  # composition of the latest steps

    # ---- adding ---------------------------------------------------------------------------------
    def _pages_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.cache.page_size)

    def add_request(self, req: InferenceRequest) -> None:
        n = req.get_prompt_length()
        if n == 0:
            self._fail(req, "empty prompt")
            return
        if n >= self.max_positions:
            self._fail(req, f"prompt of {n} tokens leaves no room under max_position_embeddings {self.max_positions}")
            return
        for g in self.cache.groups:
            if self._group_pages(g, n + 1) > g.pool.num_pages:
                self._fail(req, f"no_capacity: prompt of {n} tokens needs {self._group_pages(g, n + 1)} pages, the pool has {g.pool.num_pages}")
                return
            if self.policy == "reserve_full":
                worst = self._group_pages(g, min(n + req.sampling_params.max_tokens, self.max_positions))
                if worst > g.pool.num_pages:
                    self._fail(req, f"no_capacity: prompt and max_tokens need {worst} pages, the pool has {g.pool.num_pages}")
                    return
        req.status = RequestStatus.WAITING
        self.waiting.append(req)

    def _fail(self, req: InferenceRequest, why: str) -> None:
        req.status = RequestStatus.FAILED
        req.finish_reason = FinishReason.ERROR
        req.error = why
        self.finished.append(req)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning -------------------------------------------------------------------------------
    def _fits(self, req: InferenceRequest, n: int, promised: List[int]) -> bool:
        need = self.cache.pages_needed(req.request_id, n)
        return all(p + k <= g.pool.num_free for p, k, g in zip(promised, need, self.cache.groups))

    def _promise(self, req: InferenceRequest, n: int, promised: List[int]) -> None:
        for i, k in enumerate(self.cache.pages_needed(req.request_id, n)):
            promised[i] += k

    def _group_pages(self, group, n_tokens: int) -> int:
        """Pages of `group` that a request of `n_tokens` tokens holds at most at any time.  A group that keeps a
        window gives pages back as the window passes them: a request never holds more than the window, the
        longest portion of a step, and the page in which the window's edge lies."""
        pages = self._pages_for(n_tokens)
        if group.window > 0:
            pages = min(pages, self._pages_for(group.window + min(self.chunk_size, self.max_num_batched_tokens)) + 1)
        return pages

    def _worst_case_pages(self, req: InferenceRequest) -> List[int]:
        """Pages of each group the request may still take: up to prompt + max_tokens (scheduler.py:453-495)."""
        total = min(req.get_prompt_length() + req.sampling_params.max_tokens, self.max_positions)
        out = []
        for gi, g in enumerate(self.cache.groups):
            held = sum(1 for p in self.cache.table(req.request_id, gi) if p >= 0) if self.cache.has(req.request_id) else 0
            out.append(max(0, self._group_pages(g, total) - held))
        return out

    def _can_admit(self, req: InferenceRequest, first_portion_end: int, promised: List[int],
                   shared_pages: int = 0, shared_idle: int = 0) -> bool:
        """`first_portion_end`: tokens cached after the request's first step.  `shared_pages` of them it
        takes over from published pages; `shared_idle` of those are idle now, so taking them over
        leaves that many fewer pages to give out."""
        if self.policy == "reserve_full":
            # every group by its own need (scheduler.py:453-495 has one pool; here the groups differ: all keys, a window)
            total = min(req.get_prompt_length() + req.sampling_params.max_tokens, self.max_positions)
            running = [self._worst_case_pages(r) for r in self.running]
            for gi, g in enumerate(self.cache.groups):
                need = self._group_pages(g, total) + sum(w[gi] for w in running) - shared_pages + shared_idle
                if need > g.pool.num_free:
                    return False
            return True
        need = self._pages_for(first_portion_end) - shared_pages + shared_idle
        return all(p + need <= g.pool.num_free for p, g in zip(promised, self.cache.groups))

    def _preempt(self, victim: InferenceRequest, out: SchedulerOutput) -> None:
        self.cache.release(victim.request_id)
        self.running.remove(victim)
        victim.num_computed_tokens = 0
        victim.status = RequestStatus.WAITING
        victim.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        out.preempted.append(victim)

    def _steady_decode(self) -> Optional[SchedulerOutput]:
        """The plan of a step in which every running request decodes one token and nothing else can
        happen (nobody can be admitted, and the pools hold a page for each request in case it starts
        one): the same plan as the full procedure gives, without its page arithmetic."""
        running = self.running
        R = len(running)
        if R == 0 or R > self.max_num_batched_tokens or (self.waiting and R < self.max_num_seqs):
            return None
        for g in self.cache.groups:
            if g.pool.num_free < R:
                return None
        out = SchedulerOutput(decode_only=True)
        entries = out.entries
        for req in running:            # `running` is in order of admission
            start = req.num_computed_tokens
            if req.num_known_tokens() - start != 1 or not req.output_token_ids:
                return None
            entries.append(ScheduledEntry(req, start, 1, True))
        self.log.append({"decode": R, "portions": [], "preempted": 0,
                         "free_pages": [g.pool.num_free for g in self.cache.groups]})
        return out

    def schedule(self) -> SchedulerOutput:
        steady = self._steady_decode()
        return steady if steady is not None else self._schedule_in_full()

    def _schedule_in_full(self) -> SchedulerOutput:
        out = SchedulerOutput()
        promised = [0] * len(self.cache.groups)
        budget = self.max_num_batched_tokens

        planned_ids = set()
        gone = set()      # requests taken out of `running` during this call

        def plan(req: InferenceRequest, n: int) -> None:
            nonlocal budget
            start = req.num_computed_tokens
            self._promise(req, n, promised)
            out.entries.append(ScheduledEntry(req, start, n, start + n == req.num_known_tokens()))
            planned_ids.add(id(req))
            budget -= n

        # 1. decode tokens of running requests, oldest first; make room by preempting the newest
        for req in sorted(self.running, key=lambda r: r.admission_index):
            if id(req) in gone:               # preempted while serving an older one
                continue
            if req.num_known_tokens() - req.num_computed_tokens != 1 or req.get_num_generated_tokens() == 0:
                continue
            if budget <= 0:
                break
            while not self._fits(req, 1, promised):
                victim = max(self.running, key=lambda r: r.admission_index)
                if victim is req and len(self.running) == 1:
                    # alone with the whole pool and still short of a page: it can never finish
                    self.cache.release(req.request_id)
                    self.running.remove(req)
                    gone.add(id(req))
                    self._fail(req, "no_capacity: the request cannot make progress with the whole pool to itself")
                    break
                planned = [e for e in out.entries if e.request is victim]
                if planned:                   # never happens for decodes planned oldest-first, kept for safety
                    out.entries.remove(planned[0])
                    planned_ids.discard(id(victim))
                self._preempt(victim, out)
                gone.add(id(victim))
                if victim is req:
                    break
            if id(req) not in gone:
                plan(req, 1)
        # 2. portions of prompts already begun (and recomputations after a preemption)
        for req in sorted(self.running, key=lambda r: r.admission_index):
            left = req.num_known_tokens() - req.num_computed_tokens
            if id(req) in planned_ids or left <= 0 or budget <= 0:
                continue
            n = min(left, self.chunk_size, budget)
            while n > 0 and not self._fits(req, n, promised):
                # take what the free pages allow; a portion may end anywhere
                free_tokens = min((g.pool.num_free - p) for g, p in zip(self.cache.groups, promised)) * self.cache.page_size
                room_in_last_page = (-self.cache.length(req.request_id)) % self.cache.page_size
                n = min(n - 1, free_tokens + room_in_last_page)
            if n > 0:
                plan(req, n)
        # 3. admissions, first come first served; the first that does not fit blocks the rest
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
            req = self.waiting[0]
            if req in out.preempted:          # just made room for an older request: wait a step
                break
            # with prefix sharing the request begins after the published pages that hold its beginning
            tokens = req.all_token_ids() if self.cache.prefix_caching else None
            hit, idle = self.cache.peek_prefix(tokens) if tokens is not None else (0, 0)
            n = min(req.num_known_tokens() - hit, self.chunk_size, budget)
            if not self._can_admit(req, hit + n, promised, hit // self.cache.page_size, idle):
                break
            self.waiting.popleft()
            req.num_computed_tokens = req.num_cached_tokens = self.cache.admit(req.request_id, tokens)
            req.status = RequestStatus.RUNNING
            req.admission_index = self._admissions
            self._admissions += 1
            self.running.append(req)
            plan(req, n)
        # 4. nothing can move although requests are running: everything waits for pages that only a
        #    preemption can free
        if not out.entries and self.running:
            victim = max(self.running, key=lambda r: r.admission_index)
            if len(self.running) == 1:
                self.cache.release(victim.request_id)
                self.running.remove(victim)
                self._fail(victim, "no_capacity: the request cannot make progress with the whole pool to itself")
            else:
                self._preempt(victim, out)
                return self._merge(out, self._schedule_in_full())
        self.log.append({"decode": sum(1 for e in out.entries if e.num_tokens == 1 and e.start > 0),
                         "portions": [e.num_tokens for e in out.entries if not (e.num_tokens == 1 and e.start > 0)],
                         "preempted": len(out.preempted), "free_pages": [g.pool.num_free for g in self.cache.groups]})
        return out

    @staticmethod
    def _merge(first: SchedulerOutput, second: SchedulerOutput) -> SchedulerOutput:
        second.preempted = first.preempted + second.preempted
        return second

    # ---- after the step -----------------------------------------------------------------------
    def update(self, out: SchedulerOutput, sampled: Dict[str, int]) -> List[InferenceRequest]:
        """Advances the requests by what ran; `sampled[request_id]` is the new token of every entry
        with `samples`.  Returns the requests that finished in this step (their pages are free)."""
        done = []
        for e in out.entries:
            req = e.request
            req.num_computed_tokens += e.num_tokens
            if not e.samples:
                continue
            tok = int(sampled[req.request_id])
            req.output_token_ids.append(tok)
            reason = self._finish_reason(req, tok)
            if reason is not None:
                req.finish_reason = reason
                req.status = RequestStatus.FINISHED
                self.cache.release(req.request_id)
                self.running.remove(req)
                self.finished.append(req)
                done.append(req)
        return done

    def _finish_reason(self, req: InferenceRequest, tok: int) -> Optional[FinishReason]:
        """python/infinilm/llm/llm.py:279-303, plus stop_token_ids and the position limit."""
        sp = req.sampling_params
        if req.get_num_generated_tokens() >= sp.max_tokens:
            return FinishReason.LENGTH
        if not sp.ignore_eos:
            if tok in req.eos_token_ids:
                return FinishReason.EOS_TOKEN
            if tok in sp.stop_token_ids:
                return FinishReason.STOP
        if req.num_known_tokens() >= self.max_positions:
            return FinishReason.LENGTH
        return None

    def abort(self, req: InferenceRequest) -> None:
        if req in self.running:
            self.cache.release(req.request_id)
            self.running.remove(req)
        elif req in self.waiting:
            self.waiting.remove(req)
        else:
            return
        req.status = RequestStatus.CANCELED
        req.finish_reason = FinishReason.CANCELED
        self.finished.append(req)

    def get_cache_stats(self) -> dict:
        s = self.cache.stats()
        s.update({"waiting": len(self.waiting), "running": len(self.running), "preemptions": self.num_preemptions})
        return s
