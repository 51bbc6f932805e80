"""The two ends of a model as parts: the token embedding (ids -> float32 residual rows) and the
output head (normed rows -> float32 logits).  Like every part they are chosen by kind and built from
parameters, so that an embedding with a norm of its own or a head that caps its logits is a class
registered beside these, not a change to the model.

Reference: csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:92 (lookup) and :115-127 (head with the
logit scale); the embedding's scale is applied at lookup here (python/infinilm/modeling_utils.py:258-263
bakes it into the table), so a tied head reads the same, unscaled table (:342-351).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import kernels
from .base import BuildContext, Param, Part
from .registry import register_embedding, register_head


class Embedding(Part):
    """forward(token_ids int32 [T]) -> float32 [T, hidden]; `table` is what a tied head may read."""
    table: torch.Tensor

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class OutputHead(Part):
    """forward(x [R, hidden]) -> float32 logits [R, vocab]; `tie(table)` makes it read an embedding's table."""
    tied: bool = False

    def tie(self, table: torch.Tensor) -> None:
        raise NotImplementedError

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


@register_embedding("scaled_lookup")
class ScaledLookup(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, scale: float, ctx: BuildContext):
        self.scale = float(scale)
        self.table = torch.empty((int(vocab_size), int(hidden_size)), dtype=ctx.dtype, device=ctx.device)

    def named_parameters(self) -> Dict[str, Param]:
        return {"weight": Param(self.table)}

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return kernels.embed(token_ids, self.table, self.scale)


@register_head("linear")
class LinearHead(OutputHead):
    """logits = scale * x W^T, float32."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float, ctx: BuildContext):
        self.scale = float(scale)
        self.weight: Optional[torch.Tensor] = torch.empty((int(vocab_size), int(hidden_size)), dtype=ctx.dtype,
                                                          device=ctx.device)
        self.tied = False

    def named_parameters(self) -> Dict[str, Param]:
        return {"weight": Param(self.weight)}

    def tie(self, table: torch.Tensor) -> None:
        if tuple(table.shape) != tuple(self.weight.shape):
            raise ValueError(f"an embedding table of {tuple(table.shape)} cannot serve a head of {tuple(self.weight.shape)}")
        self.weight = table   # one tensor, no copy
        self.tied = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return kernels.gemm(x, self.weight, None, self.scale, torch.float32)
