"""Per-request state and the result structures, after the reference's
python/infinilm/llm/request.py (RequestStatus, FinishReason :40-80, RequestOutput and
CompletionOutput :85-120, InferenceRequest :144-404)."""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import List, Optional

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    CANCELED = "canceled"
    FAILED = "failed"


class FinishReason(Enum):
    EOS_TOKEN = "eos_token"
    STOP_STRING = "stop_string"
    STOP = "stop"
    LENGTH = "length"
    CANCELED = "canceled"
    ERROR = "error"


@dataclass
class CompletionOutput:
    index: int = 0
    text: str = ""
    token_ids: List[int] = field(default_factory=list)
    finish_reason: Optional[FinishReason] = None


@dataclass
class RequestOutput:
    request_id: str
    prompt: Optional[str] = None
    prompt_token_ids: Optional[List[int]] = None
    outputs: List[CompletionOutput] = field(default_factory=list)
    finished: bool = False
    finish_reason: Optional[FinishReason] = None


class InferenceRequest:
    def __init__(self, request_id: str, prompt_token_ids: List[int], sampling_params: SamplingParams,
                 prompt: Optional[str] = None, eos_token_ids: Optional[List[int]] = None, key: int = 0):
        self.request_id = request_id
        self.prompt = prompt
        self.prompt_token_ids = list(prompt_token_ids)
        self.sampling_params = sampling_params
        self.eos_token_ids = list(eos_token_ids or [])
        self.key = key                      # stable integer for the sampler's random numbers
        self.output_token_ids: List[int] = []
        self.generated_text = ""
        self.num_computed_tokens = 0        # tokens whose keys are in the cache
        self.num_cached_tokens = 0          # of these, taken over from published pages at the last admission
        self.status = RequestStatus.WAITING
        self.finish_reason: Optional[FinishReason] = None
        self.error: Optional[str] = None
        self.admission_index = -1
        self.num_preemptions = 0

    # the tokens the model has to have seen before the next token can be sampled
    def all_token_ids(self) -> List[int]:
        return self.prompt_token_ids + self.output_token_ids

    def token_slice(self, start: int, n: int) -> List[int]:
        """all_token_ids()[start:start + n] without joining the two lists."""
        lp = len(self.prompt_token_ids)
        if start >= lp:
            return self.output_token_ids[start - lp:start - lp + n]
        if start + n <= lp:
            return self.prompt_token_ids[start:start + n]
        return self.prompt_token_ids[start:] + self.output_token_ids[:start + n - lp]

    def num_known_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    def get_prompt_length(self) -> int:
        return len(self.prompt_token_ids)

    def get_num_generated_tokens(self) -> int:
        return len(self.output_token_ids)

    def is_finished(self) -> bool:
        return self.status in (RequestStatus.FINISHED, RequestStatus.CANCELED, RequestStatus.FAILED)

    def to_request_output(self) -> RequestOutput:
        return RequestOutput(request_id=self.request_id, prompt=self.prompt,
                             prompt_token_ids=list(self.prompt_token_ids),
                             outputs=[CompletionOutput(0, self.generated_text, list(self.output_token_ids),
                                                       self.finish_reason)],
                             finished=self.is_finished(), finish_reason=self.finish_reason)
