"""Interfaces of the parts a layer is put together from.

A part is built from its `PartSpec.params` (sizes and constants) and a `BuildContext` (dtype and
device); it owns its tensors and says under which names they lie in a checkpoint.  No part knows
which model it is in.

  Norm             forward(stream)                 folds the pending branch into the residual
                                                   stream and returns the normed activations
  Mixer            cache_need() -> PagedKV | FixedState | None
                   forward(x, batch, cache_view)   x [T, hidden] -> [T, hidden]; reads what it
                                                   needs of the batch (segments, positions) and
                                                   of its cache view
  FeedForward      forward(x, batch)               x [T, hidden] -> [T, hidden]
  PositionEncoding encode_and_store(qkv, batch, view, nh, nkv, d)   called by mixers: positions into
                                                   q and k, encoded k and v into the cache
  Arrangement      forward(stream, batch, cache_view)  wires the slots around the residual stream
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional

import torch


@dataclass
class BuildContext:
    dtype: torch.dtype
    device: torch.device


class Param:
    """A named tensor of a part.  `tensor` is where the loader copies to (it may be a view into a
    fused buffer).  `keep_f32`: a tensor stored in 32-bit in the checkpoint stays 32-bit even when
    the model runs in bfloat16 (the part's kernels take both).  `neutral`: the value at which the
    tensor does nothing (1.0 for a norm's gain, 0.0 for matrices and biases); random weights may be
    drawn around it."""

    def __init__(self, tensor: torch.Tensor, keep_f32: bool = False,
                 replace: Optional[Callable[[torch.Tensor], None]] = None, neutral: float = 0.0):
        self.tensor = tensor
        self.keep_f32 = keep_f32 and replace is not None
        self._replace = replace
        self.neutral = float(neutral)

    def replace(self, t: torch.Tensor) -> None:
        self._replace(t)
        self.tensor = t


class Part:
    def named_parameters(self) -> Dict[str, Param]:
        return {}


class ResidualStream:
    """The residual stream in float32 and the branch output that is still to be added to it.
    The sum `residual += scale * pending` happens inside the next norm's kernel.  `pending` is
    [T, hidden] or, from a product that was split over K, float32 parts [P, T, hidden]."""

    def __init__(self, residual: torch.Tensor):
        self.residual = residual
        self.pending: Optional[torch.Tensor] = None
        self.pending_scale: float = 1.0

    def push(self, branch: torch.Tensor, scale: float) -> None:
        if self.pending is not None:
            raise RuntimeError("a branch is already pending; a norm must fold it first")
        self.pending = branch
        self.pending_scale = scale


@dataclass
class NormTail:
    """An offer to the part before a norm (an arrangement makes it when the norm, the part before and
    the part after all can): add your branch into `residual` yourself (times `scale`) and return a
    `DeferredNorm` instead of the branch; the norm's kernel is then not run."""
    residual: torch.Tensor      # float32 [T, hidden], updated in place
    scale: float
    weight: torch.Tensor        # the norm's weight
    eps: float


@dataclass
class DeferredNorm:
    """A norm's output up to one number a row: `x` = residual * weight in the activations' dtype, and
    partial sums of squares of the residual's rows (`sumsq` [tiles, 32]), from which the consumer
    forms 1 / sqrt(mean square + eps) and applies it to its own sums."""
    x: torch.Tensor
    sumsq: torch.Tensor
    eps: float


class Norm(Part):
    """`takes_frag_request`: forward accepts `frag=True` and then returns its rows in fragment order
    (`kernels.FragRows`) for a consumer that said `takes_frag(rows)`."""
    takes_frag_request = False

    def forward(self, stream: ResidualStream) -> torch.Tensor:
        raise NotImplementedError

    def tail(self, stream: ResidualStream, scale: float, rows: int) -> Optional[NormTail]:
        """The offer for the part before this norm, or None (see NormTail)."""
        return None


class Mixer(Part):
    """`takes_tail`: forward accepts `tail=NormTail` and may answer with a DeferredNorm."""
    takes_tail = False
    # True: forward takes every index from the batch's device tensors also in steps that hold portions of prompts
    # (never from the host copies `h_*`), so that such steps can be recorded and replayed for other requests
    records_mixed_steps = False

    def takes_frag(self, rows: int) -> bool:
        """Whether forward accepts x as `kernels.FragRows` (rows in fragment order) for a step of `rows` rows."""
        return False

    def cache_need(self):
        return None

    def forward(self, x: torch.Tensor, batch, cache_view) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    records_mixed_steps = False   # as for a mixer: nothing in forward depends on the host's view of the batch

    def takes_deferred(self, rows: int) -> bool:
        """Whether forward accepts a DeferredNorm of `rows` rows as x."""
        return False

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer's queries and keys.  A mixer holds one, calls the three methods
    below and never looks inside (tables, angles and kernels are the encoding's own), so another
    encoding is a class of its own and no change to a mixer.

      max_positions   positions from here on are refused (`check`)
      encode_and_store(qkv, batch, view, nh, nkv, d)
                      encodes `batch.positions` (or whatever of `batch` it reads) into the q and k heads
                      of the fused projection rows qkv [T, (nh + 2 nkv) d], in place, and writes the
                      encoded k and the v into the cache view (`view.k`, `view.v` at `view.slots`;
                      nothing is written when `view.slots` is None).  The write belongs here because
                      the kernel that touches k anyway does it in the same pass.
      project_encode_store(x, proj, batch, view, nh, nkv, d) -> q or None
                      optional short cut: projection, encoding and cache write in one kernel for the
                      shapes an encoding has one for; returns the encoded queries [T, nh d], or None,
                      after which the mixer runs `proj.forward(x)` and `encode_and_store`.
    An encoding that cannot be written as a change of q and k (a bias on the scores) needs a mixer
    that asks for it; the mixers here do not."""

    max_positions: int = 1 << 30

    def check(self, batch) -> None:
        if batch.max_position >= self.max_positions:
            raise ValueError(f"position {batch.max_position} is beyond the position encoding's {self.max_positions}")

    def project_encode_store(self, x, proj, batch, view, nh: int, nkv: int, d: int):
        return None

    def encode_and_store(self, qkv, batch, view, nh: int, nkv: int, d: int) -> None:
        raise NotImplementedError
