"""Per-request sampling parameters, with the reference's names and defaults
(python/infinilm/llm/sampling_params.py:9-39).  Unlike the reference, where the model path uses
engine-level values for the whole batch (python/infinilm/llm/model_runner/model_runner.py:214-219),
each request's own temperature / top_p / top_k act, and `stop_token_ids` is honoured."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 0.8
    top_k: int = 1
    max_tokens: int = 512
    stop: Optional[List[str]] = None
    stop_token_ids: Optional[List[int]] = None
    ignore_eos: bool = False
    seed: Optional[int] = None  # None: the engine's seed

    def __post_init__(self):
        if self.stop is None:
            self.stop = []
        if self.stop_token_ids is None:
            self.stop_token_ids = []
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative (0 keeps the whole vocabulary), got {self.top_k}")
        if self.max_tokens <= 0:
            raise ValueError(f"max_tokens must be positive, got {self.max_tokens}")

    @property
    def greedy(self) -> bool:
        return self.top_k == 1 or self.temperature == 0.0

    def clone(self) -> "SamplingParams":
        return SamplingParams(self.temperature, self.top_p, self.top_k, self.max_tokens, list(self.stop),
                              list(self.stop_token_ids), self.ignore_eos, self.seed)
