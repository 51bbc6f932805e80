"""Grouped-query attention over the paged cache.

Reference: csrc/layers/attention/attention.cpp:96-137 (fused qkv projection -> heads -> rotation
of q and k in place -> backend -> o_proj), backends/paged_attn.cpp:20-84 (write k, v by slot, then
attention over the pages), backends/static_attn.cpp:82-99 (the formula: head h uses kv head
h // (nh/nkv), scores * scale, causal softmax, P V).  One contract serves prompts, portions of
prompts and single decoded tokens: a token at position p sees its request's keys [lo, p].
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import kernels
from ..cache.needs import PagedKV
from ..config.spec import PartSpec
from .base import BuildContext, Mixer, Param
from .linear import FusedLinear, Linear
from .registry import build_position_encoding, register_mixer


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, qkv_bias: bool,
                 out_bias: bool, scale: float, window: int, position: PartSpec, ctx: BuildContext):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} groups")
        self.nh, self.nkv, self.d = int(num_heads), int(num_kv_heads), int(head_dim)
        self.scale = float(scale)
        self.window = int(window)
        self.qkv = FusedLinear(hidden_size, [self.nh * self.d, self.nkv * self.d, self.nkv * self.d],
                               ["q_proj", "k_proj", "v_proj"], qkv_bias, ctx)
        self.o_proj = Linear(self.nh * self.d, hidden_size, "o_proj", out_bias, ctx)
        self.position = build_position_encoding(position, ctx)
        if getattr(self.position, "head_dim", self.d) not in (0, self.d):
            raise ValueError(f"the position encoding is made for heads of {self.position.head_dim}, the mixer's have {self.d}")

    def named_parameters(self) -> Dict[str, Param]:
        out = dict(self.qkv.named_parameters())
        out.update(self.o_proj.named_parameters())
        for name, p in self.position.named_parameters().items():   # an encoding may bring tensors of its own
            out[f"position.{name}"] = p
        return out

    def cache_need(self):
        return PagedKV(self.nkv, self.d, self.window)

    takes_tail = True
    records_mixed_steps = True

    def takes_frag(self, rows: int) -> bool:
        fn = getattr(self.position, "takes_frag", None)
        return bool(fn is not None and fn(rows, self.qkv, self.nh, self.nkv, self.d))

    def forward(self, x, batch, cache_view, tail=None):
        pe = self.position
        pe.check(batch)
        qkv = None
        if batch.taps is None:   # (a dump of the rotated rows needs them in one piece)
            qkv = pe.project_encode_store(x, self.qkv, batch, cache_view, self.nh, self.nkv, self.d)
        if qkv is None:
            qkv = self.qkv.forward(x)
            pe.encode_and_store(qkv, batch, cache_view, self.nh, self.nkv, self.d)
            if batch.taps is not None:
                batch.taps.setdefault("qkv_rotated", []).append(qkv.clone())
        o = kernels.paged_attention(qkv, cache_view.k, cache_view.v, cache_view.block_tables, batch.seg_of_token,
                                    batch.positions, self.nh, self.nkv, self.d, self.scale, self.window,
                                    batch.max_total_len, batch.att_tiles, batch.att_single_rows)
        if tail is not None:   # the output projection adds into the residual stream itself, where its kernel can
            deferred = self.o_proj.forward_tail(o, tail)
            if deferred is not None:
                return deferred
        return self.o_proj.forward(o, allow_parts=True)
