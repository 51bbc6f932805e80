"""MiniCPM4 (`MiniCPMForCausalLM`): the typed configuration read from config.json's own keys and
the description of the model as parts.  This file holds everything that is specific to the
architecture; no part and no kernel knows of it.

Reference: csrc/models/minicpm4/minicpm4_for_causal_lm.cpp (model, constants :12-20,:115-120,
configuration defaults :137-164), python/infinilm/infer_engine.py:73-100 (`minicpm` is the
`minicpm4` model; bias keys), csrc/config/model_config.{hpp,cpp} (required keys, head and rotary
dims, dtype).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.errors import ConfigError
from ..config.registry import register_architecture
from ..config.spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec

_DTYPES = ("float32", "bfloat16", "float16")


def _get(raw: Dict[str, Any], key: str, typ, default=None, required=False):
    if key not in raw or raw[key] is None:
        if required:
            # message of ModelConfig::get<T>: csrc/config/model_config.hpp:29-39
            raise ConfigError(f"Key '{key}' not found in config.")
        return default
    v = raw[key]
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"Key '{key}' must be an integer, got {v!r}")
        return int(v)
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"Key '{key}' must be a number, got {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"Key '{key}' must be true or false, got {v!r}")
        return v
    return v


@dataclass
class RopeScaling:
    kind: str
    short_factor: Optional[List[float]] = None
    long_factor: Optional[List[float]] = None
    original_max_position_embeddings: Optional[int] = None
    factor: float = 1.0
    extra: Optional[dict] = None   # the other keys of a kind (llama3: low/high_freq_factor; yarn: beta_*, mscale*)


@dataclass
class MiniCPM4Config:
    model_type: str
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    max_position_embeddings: int
    head_dim: int
    rotary_dim: int
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    attention_bias: bool
    attention_output_bias: bool
    mlp_bias: bool
    scale_emb: float
    scale_depth: float
    dim_model_base: Optional[float]
    tie_word_embeddings: bool
    dtype: Optional[str]
    eos_token_ids: List[int] = field(default_factory=list)
    raw: Dict[str, Any] = field(default_factory=dict, repr=False)

    # derived constants
    @property
    def residual_scale(self) -> float:
        """scale_depth / sqrt(num_hidden_layers): minicpm4_for_causal_lm.cpp:12-20."""
        return self.scale_depth / math.sqrt(float(self.num_hidden_layers))

    @property
    def logit_scale(self) -> float:
        """dim_model_base / hidden_size, only when the key exists: minicpm4_for_causal_lm.cpp:115-120."""
        return 1.0 if self.dim_model_base is None else self.dim_model_base / float(self.hidden_size)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "MiniCPM4Config":
        model_type = raw.get("model_type", "minicpm4")
        if model_type not in ("minicpm", "minicpm4"):
            archs = raw.get("architectures") or []
            if "MiniCPMForCausalLM" not in archs:
                raise ConfigError(f"model_type {model_type!r} is not minicpm4")
        H = _get(raw, "hidden_size", int, required=True)
        L = _get(raw, "num_hidden_layers", int, required=True)
        nh = _get(raw, "num_attention_heads", int, required=True)
        nkv = _get(raw, "num_key_value_heads", int, required=True)
        I = _get(raw, "intermediate_size", int, required=True)
        V = _get(raw, "vocab_size", int, required=True)
        eps = _get(raw, "rms_norm_eps", float, required=True)
        max_pos = _get(raw, "max_position_embeddings", int, required=True)
        for k, v in (("hidden_size", H), ("num_hidden_layers", L), ("num_attention_heads", nh),
                     ("num_key_value_heads", nkv), ("intermediate_size", I), ("vocab_size", V),
                     ("max_position_embeddings", max_pos)):
            if v <= 0:
                raise ConfigError(f"Key '{k}' must be positive, got {v}")
        if eps < 0:
            raise ConfigError(f"Key 'rms_norm_eps' must not be negative, got {eps}")
        if nh % nkv != 0:
            raise ConfigError(f"num_attention_heads {nh} is not a multiple of num_key_value_heads {nkv}")
        d = _get(raw, "head_dim", int)
        if d is None:
            if H % nh != 0:
                raise ConfigError(f"hidden_size {H} is not a multiple of num_attention_heads {nh} and no head_dim is given")
            d = H // nh
        if d <= 0:
            raise ConfigError(f"Key 'head_dim' must be positive, got {d}")
        # rotary dim: csrc/config/model_config.cpp:41-57
        prf = _get(raw, "partial_rotary_factor", float, 1.0)
        if prf <= 0.0 or prf >= 1.0:
            rd = d
        else:
            rd = int(round(d * prf))
            rd = min(max(rd, 2), d)
            if rd % 2:
                rd -= 1
            rd = max(rd, 2)
        if rd % 2:
            raise ConfigError(f"the rotary dimension {rd} (head_dim {d}) must be even")
        theta = _get(raw, "rope_theta", float, 10000.0)
        scaling = cls._rope_scaling(raw.get("rope_scaling"), rd)
        # bias keys: minicpm4_for_causal_lm.cpp:150-162
        bias = _get(raw, "bias", bool)
        att_b = bias if bias is not None else _get(raw, "attention_bias", bool, False)
        mlp_b = bias if bias is not None else _get(raw, "mlp_bias", bool, False)
        out_b = _get(raw, "attention_output_bias", bool, False)
        dtype = raw.get("dtype", raw.get("torch_dtype"))
        if dtype is not None and dtype not in _DTYPES:
            raise ConfigError(f"Unsupported dtype string: {dtype}")
        eos = raw.get("eos_token_id") or []
        if isinstance(eos, int):
            eos = [eos]
        if raw.get("quantization_config") is not None:
            raise ConfigError("quantized checkpoints are not supported")
        return cls(model_type=model_type, hidden_size=H, num_hidden_layers=L, num_attention_heads=nh,
                   num_key_value_heads=nkv, intermediate_size=I, vocab_size=V, rms_norm_eps=eps,
                   max_position_embeddings=max_pos, head_dim=d, rotary_dim=rd, rope_theta=theta,
                   rope_scaling=scaling, attention_bias=att_b, attention_output_bias=out_b, mlp_bias=mlp_b,
                   scale_emb=_get(raw, "scale_emb", float, 1.0), scale_depth=_get(raw, "scale_depth", float, 1.0),
                   dim_model_base=_get(raw, "dim_model_base", float),
                   tie_word_embeddings=_get(raw, "tie_word_embeddings", bool, False),
                   dtype=dtype, eos_token_ids=[int(e) for e in eos], raw=dict(raw))

    @staticmethod
    def _rope_scaling(rs, rd: int) -> Optional[RopeScaling]:
        """csrc/layers/rotary_embedding/rotary_embedding_factory.cpp:11-39 and
        rope_scaling_creators.cpp:23-47."""
        if rs is None:
            return None
        if not isinstance(rs, dict):
            raise ConfigError("rope_scaling must be an object")
        kind = rs.get("type", rs.get("rope_type"))
        if kind is None:
            raise ConfigError("rope_scaling must contain 'type' or 'rope_type' field")
        if kind in ("default", "none", "dynamic"):
            return None
        if kind == "llama3":   # rope_scaling_creators.cpp:54-75
            need = ("factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings")
            if any(k not in rs for k in need):
                raise ConfigError("Llama3RopeScalingConfig requires 'factor', 'low_freq_factor', 'high_freq_factor', and "
                                  "'original_max_position_embeddings'")
            if float(rs["high_freq_factor"]) <= float(rs["low_freq_factor"]) or float(rs["factor"]) <= 0:
                raise ConfigError("llama3 rope scaling needs factor > 0 and high_freq_factor > low_freq_factor")
            return RopeScaling("llama3", None, None, int(rs["original_max_position_embeddings"]), float(rs["factor"]),
                               {"low_freq_factor": float(rs["low_freq_factor"]), "high_freq_factor": float(rs["high_freq_factor"])})
        if kind == "yarn":     # rope_scaling_creators.cpp:80-102 (keys and their defaults)
            if "factor" not in rs or "original_max_position_embeddings" not in rs:
                raise ConfigError("YarnRopeScalingConfig requires 'factor' and 'original_max_position_embeddings'")
            if float(rs["factor"]) <= 0:
                raise ConfigError("yarn rope scaling needs factor > 0")
            return RopeScaling("yarn", None, None, int(rs["original_max_position_embeddings"]), float(rs["factor"]),
                               {"beta_fast": int(float(rs.get("beta_fast", 32.0))), "beta_slow": int(float(rs.get("beta_slow", 1.0))),
                                "mscale": float(rs.get("mscale", 1.0)), "mscale_all_dim": float(rs.get("mscale_all_dim", 0.0))})
        if kind != "longrope":
            raise ConfigError(f"Unsupported rope_scaling_type: {kind}")
        for k in ("short_factor", "long_factor", "original_max_position_embeddings"):
            if k not in rs:
                raise ConfigError("LongRopeConfig requires 'short_factor', 'long_factor', and "
                                  "'original_max_position_embeddings'")
        short = [float(x) for x in rs["short_factor"]]
        long = [float(x) for x in rs["long_factor"]]
        if len(short) != rd // 2 or len(long) != rd // 2:
            raise ConfigError(f"short_factor ({len(short)}) and long_factor ({len(long)}) must have "
                              f"rotary_dim/2 = {rd // 2} entries")
        if any(x <= 0 for x in short + long):
            raise ConfigError("rope scaling factors must be positive")
        orig = int(rs["original_max_position_embeddings"])
        if orig <= 1:
            raise ConfigError("original_max_position_embeddings must be above 1")
        return RopeScaling("longrope", short, long, orig, float(rs.get("factor", 1.0)))


def build_spec(cfg: MiniCPM4Config) -> ModelSpec:
    """embed*scale_emb -> L x (norm, GQA attention * a, norm, SwiGLU * a) -> norm -> head * (base/H),
    a = scale_depth / sqrt(L): minicpm4_for_causal_lm.cpp:49-57,89-101,123-127."""
    scaling = None
    if cfg.rope_scaling is not None:
        s = cfg.rope_scaling
        scaling = {"type": s.kind, "original_max_position_embeddings": s.original_max_position_embeddings, "factor": s.factor}
        if s.kind == "longrope":
            scaling.update(short_factor=s.short_factor, long_factor=s.long_factor)
        scaling.update(s.extra or {})
    position = PartSpec("rotary", {"head_dim": cfg.head_dim, "rotary_dim": cfg.rotary_dim,
                                   "max_positions": cfg.max_position_embeddings, "theta": cfg.rope_theta,
                                   "scaling": scaling})
    mixer = PartSpec("gqa_attention", {
        "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
        "qkv_bias": cfg.attention_bias, "out_bias": cfg.attention_output_bias,
        "scale": 1.0 / math.sqrt(cfg.head_dim),  # attention.cpp:41
        "window": 0, "position": position})
    ffn = PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                              "bias": cfg.mlp_bias})
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layers = [LayerSpec(prefix=f"model.layers.{i}", arrangement="pre_norm",
                        parts={"norm1": norm, "mixer": mixer, "norm2": norm, "ffn": ffn},
                        names={"norm1": "input_layernorm", "mixer": "self_attn",
                               "norm2": "post_attention_layernorm", "ffn": "mlp"},
                        residual_scale=cfg.residual_scale)
              for i in range(cfg.num_hidden_layers)]
    order = [LayerRun(layer=i, cache=i, writes_cache=True) for i in range(cfg.num_hidden_layers)]
    spec = ModelSpec(architecture="MiniCPMForCausalLM", vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                     max_positions=cfg.max_position_embeddings, embed_name="model.embed_tokens",
                     embed_scale=cfg.scale_emb, layers=layers, order=order, final_norm=norm,
                     final_norm_name="model.norm",
                     head=HeadSpec(name="lm_head", scale=cfg.logit_scale, tie_to_embedding_when_missing=True),
                     eos_token_ids=list(cfg.eos_token_ids))
    spec.validate()
    return spec


register_architecture(["MiniCPMForCausalLM", "minicpm4", "minicpm"], MiniCPM4Config.from_dict, build_spec)
