"""From rows of logits to tokens: argmax for greedy rows, temperature / top-k / top-p otherwise.

Reference: one `random_sample_(out, row, random_val, top_p, top_k, temperature)` call per request
in a host loop, random_val from a `std::mt19937` seeded by `std::random_device`
(csrc/engine/rank_worker.cpp:27,467-513): not reproducible.  Here all rows are sampled by one
kernel launch, and the uniform number of a row is a pure function of (seed, request, index of the
generated token), so a request's tokens do not depend on what else is in the batch or on how often
it was preempted.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np
import torch

from .. import kernels
from .params import SamplingParams

_MASK = (1 << 64) - 1


def _mix(x: int) -> int:
    """splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D2049BB133111B) & _MASK
    return x ^ (x >> 31)


def uniform_for(seed: int, request_key: int, index: int) -> float:
    """u in [0, 1) with 24 bits, a pure function of its arguments."""
    x = _mix(_mix(_mix(seed & _MASK) ^ (request_key & _MASK)) ^ (index & _MASK))
    return (x >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, seed: int = 0):
        self.seed = int(seed)
        # pinned host memory for the rows' parameters: two buffers in turn, each waited for only when
        # its own last copy may still be reading it (a step may be launched before the one before it
        # has run)
        self._staging = [None, None]
        self._copied = [None, None]
        self._turn = 0

    def sample(self, logits: torch.Tensor, rows: Sequence[Tuple[SamplingParams, int, int]]) -> List[int]:
        """`rows[i]` = (params, request key, index of the token being generated) for logits[i]."""
        if logits.shape[0] == 0 and not rows:
            return []
        return self.sample_device(logits, rows).tolist()

    def sample_device(self, logits: torch.Tensor, rows: Sequence[Tuple[SamplingParams, int, int]]) -> torch.Tensor:
        """The same, the tokens left on the device (int32 [rows]); nothing waits for the stream."""
        n = logits.shape[0]
        if n != len(rows):
            raise ValueError(f"{n} rows of logits for {len(rows)} requests")
        if n == 0:
            raise ValueError("no rows to sample")
        if all(p.greedy for p, _, _ in rows):
            return kernels.argmax(logits)
        # temperature, top_k, top_p and the uniform numbers in one pinned buffer and one copy that
        # queues behind the step (a copy from pageable memory would make the host wait for the step
        # and the device wait for four copies)
        dev = logits.device
        t = self._turn = self._turn ^ 1
        if self._copied[t] is not None:
            self._copied[t].synchronize()
            self._copied[t] = None
        if self._staging[t] is None or self._staging[t].numel() < 4 * n:
            self._staging[t] = torch.empty((4 * max(n, 64),), dtype=torch.float32, pin_memory=dev.type == "cuda")
        host = self._staging[t][:4 * n]
        h = host.numpy()
        h[0:n] = [p.temperature for p, _, _ in rows]
        h[n:2 * n].view(np.int32)[:] = [p.top_k for p, _, _ in rows]
        h[2 * n:3 * n] = [p.top_p for p, _, _ in rows]
        h[3 * n:4 * n] = [uniform_for(self.seed if p.seed is None else p.seed, key, idx) for p, key, idx in rows]
        d = torch.empty((4 * n,), dtype=torch.float32, device=dev)
        d.copy_(host, non_blocking=True)
        if dev.type == "cuda":
            self._copied[t] = torch.cuda.Event()
            self._copied[t].record()
        return kernels.sample(logits, d[0:n], d[n:2 * n].view(torch.int32), d[2 * n:3 * n], d[3 * n:4 * n])
