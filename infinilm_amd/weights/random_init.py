"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a
seed, and an in-place fill of a built model on its device for runs too large to pass through a file.

The reference's `--skip-load` leaves device memory uninitialised
(python/infinilm/llm/model_runner/model_runner.py:104-107); here weights are always drawn:
every tensor N(0, std) from a generator seeded with (seed, position of the tensor in name order);
`norm_init="one_plus"` draws the tensors whose part declares a neutral value (`Param.neutral`: 1 for
a norm's gain) as neutral + N(0, std), so that deep random models keep activations of order one.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

_TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def _describe(config: dict):
    from ..config.registry import load_model_config
    from ..engine.model import CausalLM

    arch, cfg = load_model_config(config)
    spec = arch.build_spec(cfg)
    return cfg, CausalLM(spec, torch.float32, "meta")


def random_state_dict(config: dict, seed: int, std: float = 0.02, norm_init: str = "normal",
                      dtype: Optional[str] = None) -> Dict[str, torch.Tensor]:
    cfg, meta = _describe(config)
    store = _TORCH_DTYPES[dtype or config.get("torch_dtype", config.get("dtype", "float32"))]
    tied = bool(config.get("tie_word_embeddings", False))
    out: Dict[str, torch.Tensor] = {}
    for i, (name, p) in enumerate(sorted(meta.named_parameters().items())):
        if tied and name == f"{meta.spec.head.name}.weight":
            continue
        g = torch.Generator().manual_seed((int(seed) * 1000003 + i) & 0x7fffffffffff)
        t = torch.randn(tuple(p.tensor.shape), generator=g, dtype=torch.float32) * std
        if norm_init == "one_plus" and p.neutral != 0.0:
            t = t + p.neutral
        out[name] = t.to(store).contiguous()
    return out


def write_random_model(config: dict, seed: int, out_dir: str, std: float = 0.02, norm_init: str = "normal",
                       dtype: Optional[str] = None) -> str:
    """Writes out_dir/config.json and out_dir/model.safetensors; returns out_dir."""
    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    sd = random_state_dict(config, seed, std, norm_init, dtype)
    cfg = dict(config)
    if dtype is not None:
        cfg["torch_dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(cfg, fh, indent=1)
    save_file(sd, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    return out_dir


def fill_random_(model, seed: int, std: float = 0.02, norm_init: str = "one_plus", tie: bool = False) -> None:
    """Draws every parameter of a built model on its own device (no file, no host copy)."""
    if tie:
        model.tie_head_to_embedding()
    g = torch.Generator(device=model.device).manual_seed(int(seed))
    done = set()
    for name, p in sorted(model.named_parameters().items()):
        t = p.tensor
        key = (t.data_ptr(), tuple(t.shape))
        if key in done:
            continue
        done.add(key)
        # draw in slabs so that a large matrix needs no float32 copy of itself
        flat = t.view(-1) if t.is_contiguous() else None
        if flat is None:
            t.copy_((torch.randn(t.shape, generator=g, device=t.device, dtype=torch.float32) * std).to(t.dtype))
        else:
            step = 1 << 26
            for a in range(0, flat.numel(), step):
                b = min(flat.numel(), a + step)
                flat[a:b] = (torch.randn((b - a,), generator=g, device=t.device, dtype=torch.float32) * std).to(t.dtype)
        if norm_init == "one_plus" and p.neutral != 0.0:
            t.add_(p.neutral)
