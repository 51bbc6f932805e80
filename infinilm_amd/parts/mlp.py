"""SwiGLU feed-forward: down(silu(gate x) * up x).

Reference: csrc/layers/mlp/mlp.cpp:7-38; gate and up are the two halves (gate first) of one fused
projection: csrc/layers/linear/fused_linear.cpp:152-158,177-180.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels
from .base import BuildContext, DeferredNorm, FeedForward, Param
from .linear import FusedLinear, Linear
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    records_mixed_steps = True

    def __init__(self, hidden_size: int, intermediate_size: int, bias: bool, ctx: BuildContext):
        self.gate_up = FusedLinear(hidden_size, [intermediate_size, intermediate_size], ["gate_proj", "up_proj"],
                                   bias, ctx)
        self.down = Linear(intermediate_size, hidden_size, "down_proj", bias, ctx)

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.gate_up.named_parameters())
        out.update(self.down.named_parameters())
        return out

    def takes_deferred(self, rows: int) -> bool:
        return kernels.gateup_resident_ok(rows, self.gate_up.weight)

    def forward(self, x, batch) -> torch.Tensor:
        if isinstance(x, DeferredNorm):   # the norm's division happens in the gate/up kernel's epilogue
            act = kernels.gateup_swiglu_gemm(x.x, self.gate_up.weight, self.gate_up.bias, row_ss=x.sumsq, eps=x.eps)
            return self.down.forward(act, allow_parts=True)
        frag = (lambda: self.gate_up.frag_weight("gate_up8")) if kernels.frag_weight_ok(self.gate_up.weight) else None
        act = kernels.gateup_swiglu_gemm(x, self.gate_up.weight, self.gate_up.bias, frag_w=frag)   # few rows: activation in the epilogue
        if act is not None:
            return self.down.forward(act, allow_parts=True)
        gu = self.gate_up.forward(x)
        if self.down.bias is None:
            fused = kernels.swiglu_gemm(gu, self.down.weight)   # few rows: activation inside the product
            if fused is not None:
                return fused
        return self.down.forward(kernels.swiglu(gu), allow_parts=True)
