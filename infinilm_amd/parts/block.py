"""Arrangements: how a layer's parts are wired around the residual stream.

`pre_norm`: x += s * mixer(norm1(x)); x += s * ffn(norm2(x)), the reference's decoder layer
(csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:49-71, csrc/layers/causal_lm_templates/
text_decoder_layer.hpp:39-61).  The adds are deferred into the next norm's kernel.
"""
from __future__ import annotations

from typing import Dict

from ..config.spec import LayerSpec
from .base import BuildContext, DeferredNorm, Param, ResidualStream
from .registry import ARRANGEMENTS, build_feed_forward, build_mixer, build_norm, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    slots = ("norm1", "mixer", "norm2", "ffn")

    def __init__(self, spec: LayerSpec, ctx: BuildContext):
        self.spec = spec
        self.norm1 = build_norm(spec.parts["norm1"], ctx)
        self.mixer = build_mixer(spec.parts["mixer"], ctx)
        self.norm2 = build_norm(spec.parts["norm2"], ctx)
        self.ffn = build_feed_forward(spec.parts["ffn"], ctx)
        self.residual_scale = float(spec.residual_scale)

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for slot in self.slots:
            sub = self.spec.names[slot]
            for name, p in getattr(self, slot).named_parameters().items():
                out[f"{self.spec.prefix}.{sub}.{name}"] = p
        return out

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def records_mixed_steps(self) -> bool:
        return bool(getattr(self.mixer, "records_mixed_steps", False) and getattr(self.ffn, "records_mixed_steps", False))

    def forward(self, stream: ResidualStream, batch, cache_view) -> None:
        # a decode step of many rows: the mixer may take its rows in fragment order, which the norm then writes
        rows = stream.residual.shape[0]
        if (batch.taps is None and getattr(self.norm1, "takes_frag_request", False)
                and getattr(self.mixer, "takes_frag", lambda rows: False)(rows)):
            x = self.norm1.forward(stream, frag=True)
        else:
            x = self.norm1.forward(stream)
        # Few rows (decoded tokens): where the mixer's last projection, the second norm and the feed-forward
        # all can, the projection adds into the residual stream itself and the norm's kernel is not run
        # (see NormTail).  Not while intermediate values are dumped: they are taken between the kernels.
        tail = None
        if self.mixer.takes_tail and batch.taps is None:
            tail = self.norm2.tail(stream, self.residual_scale, x.shape[0])
            if tail is not None and not self.ffn.takes_deferred(x.shape[0]):
                tail = None
        y = self.mixer.forward(x, batch, cache_view) if tail is None else self.mixer.forward(x, batch, cache_view, tail=tail)
        if isinstance(y, DeferredNorm):
            x = y
        else:
            stream.push(y, self.residual_scale)
            x = self.norm2.forward(stream)
        stream.push(self.ffn.forward(x, batch), self.residual_scale)


def build_block(spec: LayerSpec, ctx: BuildContext):
    try:
        cls = ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown arrangement {spec.arrangement!r}; registered: {sorted(ARRANGEMENTS)}") from None
    return cls(spec, ctx)
