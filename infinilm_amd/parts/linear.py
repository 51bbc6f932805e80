"""Dense projections y = alpha * (x W^T + b), W [out, in].

Reference: csrc/layers/linear/base_linear.{hpp,cpp} (alpha, weight layout) and fused_linear.cpp
(:62-71 the q|k|v split, :90-111 and :163-185 the named row-slices of one fused weight): several
checkpoint tensors are row ranges of one allocation, so loading by name fills the fused weight and
one product computes all of them.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .. import kernels
from .base import BuildContext, DeferredNorm, NormTail, Param


class FusedLinear:
    """`out_sizes[i]` rows of the weight belong to the checkpoint tensor `names[i]`."""

    def __init__(self, in_features: int, out_sizes: Sequence[int], names: Sequence[str], bias: bool,
                 ctx: BuildContext):
        self.in_features = int(in_features)
        self.out_sizes = [int(s) for s in out_sizes]
        self.names = list(names)
        n = sum(self.out_sizes)
        self.weight = torch.empty((n, self.in_features), dtype=ctx.dtype, device=ctx.device)
        self.bias = torch.empty((n,), dtype=ctx.dtype, device=ctx.device) if bias else None
        self._frag = {}   # layout -> (version of the weight it was packed from, the weight in fragment order)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        row = 0
        for name, size in zip(self.names, self.out_sizes):
            out[f"{name}.weight"] = Param(self.weight[row:row + size])
            if self.bias is not None:
                out[f"{name}.bias"] = Param(self.bias[row:row + size])
            row += size
        return out

    def frag_weight(self, kind: str = "plain", **layout):
        """The weight in fragment order (`kernels.pack_weight`), packed at its first use and again when the weight
        has been written since (a second copy of the weight: the many-rows products keep the plain rows)."""
        key = (kind, tuple(sorted(layout.items())))
        held = self._frag.get(key)
        if held is None or held[0] != self.weight._version or held[2] != self.weight.data_ptr():
            held = (self.weight._version, kernels.pack_weight(self.weight, kind, **layout), self.weight.data_ptr())
            self._frag[key] = held
        return held[1]

    def forward(self, x: torch.Tensor, alpha: float = 1.0, out_dtype: Optional[torch.dtype] = None,
                allow_parts: bool = False) -> torch.Tensor:
        """`allow_parts`: the result may come as float32 parts [P, T, out] still to be summed; only for a
        result that goes straight into `ResidualStream.push` (the next norm's kernel sums them)."""
        frag = self.frag_weight if kernels.frag_weight_ok(self.weight) and x.shape[0] <= max(kernels.FRAG_MAX_ROWS, kernels.TALL_MAX_ROWS) else None
        return kernels.gemm(x, self.weight, self.bias, alpha, out_dtype, allow_parts=allow_parts, frag_w=frag)


    def forward_tail(self, x: torch.Tensor, tail: NormTail) -> Optional[DeferredNorm]:
        """The projection with the residual sum and the first half of the following norm in its epilogue
        (`kernels.gemm_tail`), or None where that kernel does not take the shapes."""
        if not kernels.tail_ok(x.shape[0], self.weight, self.bias, tail.weight, x.dtype):
            return None
        xw, ss = kernels.gemm_tail(x, self.weight, self.bias, tail.scale, tail.residual, tail.weight)
        return DeferredNorm(xw, ss, tail.eps)


class Linear(FusedLinear):
    def __init__(self, in_features: int, out_features: int, name: str, bias: bool, ctx: BuildContext):
        super().__init__(in_features, [out_features], [name], bias, ctx)
