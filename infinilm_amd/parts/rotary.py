"""Rotary position encoding with its scaling kinds.

Reference: csrc/layers/rotary_embedding/rotary_embedding.cpp:90-113 (one table for
max_position_embeddings positions, shared by the layers), rotary_embedding_factory.cpp:11-39 (kind
from `type` or `rope_type`; absent/null = none), rope_scaling_creators.cpp:23-47,106-115 (longrope's
keys; `default`, `none`, `dynamic` = no scaling; `llama3` and `yarn` below), csrc/config/model_config.hpp:139 (rotate-half
pairing).  The arithmetic is the tensor library's in the reference; the definition used:

  inv_freq_i = 1 / (f_i * theta^(2i/rd)),  i < rd/2
  longrope: f = long_factor if max_positions > original_max else short_factor (the table is built
            once, before any request, so the choice cannot depend on a request's length);
            s = factor if given and != 1 else max_positions/original_max;
            m = sqrt(1 + ln s / ln original_max) if s > 1 else 1
  cos = m cos(p inv_freq), sin = m sin(p inv_freq), angles in float64, tables stored in float32.
"""
from __future__ import annotations

import inspect
import math
from typing import Callable, Dict, Optional, Tuple

import torch

from .. import kernels
from .base import BuildContext, PositionEncoding
from .registry import register_position_encoding

# kind -> function(inv_freq float64 [rd/2], params, max_positions[, theta=base]) -> (inv_freq, magnitude)
SCALINGS: Dict[str, Callable] = {}


def register_rope_scaling(kind: str):
    def deco(fn):
        SCALINGS[kind] = fn
        return fn
    return deco


@register_rope_scaling("default")
@register_rope_scaling("none")
@register_rope_scaling("dynamic")
def _no_scaling(inv_freq, params, max_positions):
    return inv_freq, 1.0


@register_rope_scaling("longrope")
def _longrope(inv_freq, params, max_positions):
    orig = int(params["original_max_position_embeddings"])
    factors = params["long_factor"] if max_positions > orig else params["short_factor"]
    f = torch.tensor(factors, dtype=torch.float64)
    if f.numel() != inv_freq.numel():
        raise ValueError(f"longrope factors have {f.numel()} entries, the rotary dimension needs {inv_freq.numel()}")
    s = float(params.get("factor", 1.0) or 1.0)
    if s == 1.0:
        s = max_positions / orig
    m = math.sqrt(1.0 + math.log(s) / math.log(orig)) if s > 1.0 else 1.0
    return inv_freq / f, m


@register_rope_scaling("llama3")
def _llama3(inv_freq, params, max_positions, theta=None):
    """Keys: rope_scaling_creators.cpp:54-75 (factor, low_freq_factor, high_freq_factor,
    original_max_position_embeddings).  The arithmetic is in the reference's tensor library, not in its
    text (parity unpinned); the definition used, with wavelength 2 pi / inv_freq and o the original length:
      wavelength < o / high_freq_factor  ->  unchanged
      wavelength > o / low_freq_factor   ->  inv_freq / factor
      between: s = (o / wavelength - low_freq_factor) / (high_freq_factor - low_freq_factor),
               inv_freq * ((1 - s) / factor + s)."""
    factor, lo, hi = float(params["factor"]), float(params["low_freq_factor"]), float(params["high_freq_factor"])
    orig = float(params["original_max_position_embeddings"])
    wavelen = 2.0 * math.pi / inv_freq
    s = ((orig / wavelen - lo) / (hi - lo)).clamp(0.0, 1.0)   # 0 below the low band's edge, 1 above the high one's
    return inv_freq * ((1.0 - s) / factor + s), 1.0


@register_rope_scaling("yarn")
def _yarn(inv_freq, params, max_positions, theta=None):
    """Keys and defaults: rope_scaling_creators.cpp:80-102 (factor, original_max_position_embeddings,
    beta_fast 32, beta_slow 1, mscale 1, mscale_all_dim 0; rotary dim and rope_theta from the model).
    The arithmetic is in the reference's tensor library, not in its text (parity unpinned); the
    definition used, with D the rotary dim, b = theta and o the original length:
      c(beta) = D ln(o / (2 pi beta)) / (2 ln b)            the pair index that turns beta times within o
      lo = max(floor(c(beta_fast)), 0), hi = min(ceil(c(beta_slow)), D/2 - 1)
      ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)   0: turns often, kept; 1: turns seldom, stretched
      inv_freq_i * (1 - ramp_i) + inv_freq_i / factor * ramp_i
      magnitude = g(mscale) / g(mscale_all_dim), g(m) = 0.1 m ln(factor) + 1 for factor > 1, else 1."""
    factor, orig = float(params["factor"]), float(params["original_max_position_embeddings"])
    half = inv_freq.numel()
    D = 2 * half
    base = float(theta if theta is not None else params.get("rope_theta", 10000.0))
    corr = lambda beta: D * math.log(orig / (2.0 * math.pi * beta)) / (2.0 * math.log(base))
    lo = max(math.floor(corr(float(params.get("beta_fast", 32)))), 0)
    hi = min(math.ceil(corr(float(params.get("beta_slow", 1)))), half - 1)
    i = torch.arange(half, dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    g = lambda m: 0.1 * m * math.log(factor) + 1.0 if factor > 1.0 else 1.0
    return inv_freq * (1.0 - ramp) + inv_freq / factor * ramp, g(float(params.get("mscale", 1.0))) / g(float(params.get("mscale_all_dim", 0.0)))


_TABLE_CACHE: Dict[Tuple, Tuple[torch.Tensor, torch.Tensor]] = {}


@register_position_encoding("rotary")
class RotaryEmbedding(PositionEncoding):
    """Tables cos/sin [max_positions, rotary_dim/2] float32; layers with equal parameters share them."""

    def __init__(self, head_dim: int, rotary_dim: int, max_positions: int, theta: float,
                 scaling: Optional[dict], ctx: BuildContext):
        if rotary_dim % 2 or rotary_dim > head_dim or rotary_dim < 0:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim}")
        self.head_dim, self.rotary_dim, self.max_positions = int(head_dim), int(rotary_dim), int(max_positions)
        self.theta = float(theta)
        self.scaling = scaling
        key = (self.rotary_dim, self.max_positions, self.theta, repr(scaling), str(ctx.device))
        if key not in _TABLE_CACHE:
            cos, sin = self._build()
            _TABLE_CACHE[key] = (cos.to(ctx.device), sin.to(ctx.device))
        self.cos, self.sin = _TABLE_CACHE[key]

    def _build(self):
        rd = self.rotary_dim
        i = torch.arange(rd // 2, dtype=torch.float64)
        inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), 2.0 * i / max(rd, 1))
        m = 1.0
        if self.scaling is not None:
            kind = self.scaling.get("type", self.scaling.get("rope_type"))
            if kind not in SCALINGS:
                raise ValueError(f"Unsupported rope_scaling_type: {kind}")
            fn = SCALINGS[kind]
            # a scaling that names a `theta` parameter (or takes any keyword) is given the base theta by
            # keyword (yarn's band edges need it); the signature is looked at, not the code object, so
            # partials and wrapped callables work too
            try:
                params = inspect.signature(fn).parameters
                takes_theta = "theta" in params or any(p.kind is p.VAR_KEYWORD for p in params.values())
            except (TypeError, ValueError):
                takes_theta = False
            if takes_theta:
                inv_freq, m = fn(inv_freq, self.scaling, self.max_positions, theta=self.theta)
            else:
                inv_freq, m = fn(inv_freq, self.scaling, self.max_positions)
        p = torch.arange(self.max_positions, dtype=torch.float64)
        ang = p[:, None] * inv_freq[None, :]
        return (torch.cos(ang) * m).to(torch.float32).contiguous(), (torch.sin(ang) * m).to(torch.float32).contiguous()

    def takes_frag(self, rows, proj, nh, nkv, d):
        return kernels.qkv_frag_ok(rows, proj.weight, d, self.rotary_dim, proj.in_features)

    def project_encode_store(self, x, proj, batch, view, nh, nkv, d):
        # few rows (decoded tokens): projection, rotation and cache write are one kernel
        if isinstance(x, kernels.FragRows):   # rows in fragment order, as `takes_frag` offered
            return kernels.gemm_frag_rope(x, proj.frag_weight("qkv", nh=nh, nkv=nkv, d=d), proj.bias, batch.positions,
                                          self.cos, self.sin, view.k, view.v, view.slots, nh, nkv, d)
        return kernels.qkv_rope_gemm(x, proj.weight, proj.bias, batch.positions, self.cos, self.sin, view.k, view.v,
                                     view.slots, nh, nkv, d, self.rotary_dim)

    def encode_and_store(self, qkv, batch, view, nh, nkv, d):
        kernels.rope_kvwrite(qkv, batch.positions, self.cos, self.sin, view.k, view.v, view.slots, nh, nkv, d,
                             self.rotary_dim)


@register_position_encoding("none")
class NoPositionEncoding(RotaryEmbedding):
    """No rotation (a rotary encoding over no dims): keys and values go to the cache as they are."""

    def __init__(self, ctx: BuildContext, head_dim: int = 0, **_):
        self.head_dim, self.rotary_dim, self.max_positions = int(head_dim), 0, 1 << 30
        self.cos = torch.zeros((1, 0), dtype=torch.float32, device=ctx.device)
        self.sin = torch.zeros((1, 0), dtype=torch.float32, device=ctx.device)

    def takes_frag(self, rows, proj, nh, nkv, d):
        return False

    def project_encode_store(self, x, proj, batch, view, nh, nkv, d):
        return None
