"""RMS norm fused with the residual add.

Reference: `RMSNorm::forward_inplace(h, residual)` as used in
csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:52,54,99: residual = h + residual, h = norm(residual).
Here the residual stream is float32 and the branch's scale (the reference's GEMM alpha on o_proj
and down_proj, :23-34) is applied in the same kernel: residual += scale * branch.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels
from .base import BuildContext, Norm, NormTail, Param, ResidualStream
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    takes_frag_request = True

    def __init__(self, size: int, eps: float, ctx: BuildContext):
        self.size = int(size)
        self.eps = float(eps)
        self.dtype = ctx.dtype
        self.weight = torch.empty((self.size,), dtype=ctx.dtype, device=ctx.device)

    def _set_weight(self, t: torch.Tensor) -> None:
        self.weight = t

    def named_parameters(self) -> Dict[str, Param]:
        return {"weight": Param(self.weight, keep_f32=True, replace=self._set_weight, neutral=1.0)}

    def tail(self, stream: ResidualStream, scale: float, rows: int):
        if stream.pending is not None or self.dtype != torch.bfloat16 or rows > kernels.TAIL_MAX_ROWS:
            return None
        return NormTail(stream.residual, float(scale), self.weight, self.eps)

    def forward(self, stream: ResidualStream, frag: bool = False):
        """`frag`: the consumer takes its rows in fragment order (`kernels.FragRows`)."""
        x = kernels.add_rmsnorm(stream.residual, stream.pending, self.weight, stream.pending_scale, self.eps,
                                self.dtype, frag=frag)
        stream.pending = None
        stream.pending_scale = 1.0
        return x
