"""Weights from safetensors, by tensor name.

Reference: python/infinilm/modeling_utils.py:192-359: `model.safetensors.index.json` first, else
every `*.safetensors` of the folder (:222-236,:296-340); tensors go to the parameter of the same
name; a checkpoint without `lm_head.weight` makes the head use the (unscaled) embedding table
(:342-351); one check at the end reports missing and unexpected names (:71-100,:353).
Here: the embedding's scale is applied at lookup, not baked into the table (:258-263 bakes it), so
a tied head aliases the table instead of holding a second copy; wrong shapes are part of the same
single error.

Dtypes: matrices are kept in the run dtype (bfloat16 in serving, everything float32 on the 32-bit
path); integer tables become int32; a tensor the checkpoint stores in 32-bit stays 32-bit where
the owning part can take it (`Param.keep_f32`, e.g. norm weights).
"""
from __future__ import annotations

import glob
import json
import os
from typing import Iterator, List, Tuple

import torch


class WeightError(RuntimeError):
    """Missing, unexpected or wrongly shaped tensors; lists all of them."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[str], other: List[str] = ()):
        self.missing, self.unexpected, self.wrong_shape, self.other = list(missing), list(unexpected), list(wrong_shape), list(other)
        parts = ["Error(s) in loading weights:"]
        if self.missing:
            parts.append(f"  Missing tensor(s) ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            parts.append(f"  Unexpected tensor(s) ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            parts.append(f"  Wrong shape(s) ({len(self.wrong_shape)}): " + "; ".join(self.wrong_shape))
        if self.other:
            parts.append("  " + "; ".join(self.other))
        super().__init__("\n".join(parts))


def weight_files(model_dir: str) -> List[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as fh:
            names = sorted(set(json.load(fh)["weight_map"].values()))
        return [os.path.join(model_dir, n) for n in names]
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"Weight file not found: no *.safetensors in {model_dir}")
    return files


def iter_tensors(model_dir: str) -> Iterator[Tuple[str, torch.Tensor]]:
    from safetensors import safe_open

    for path in weight_files(model_dir):
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)


def load_weights(model, model_dir: str) -> None:
    """Fills `model`'s parameters from the folder's safetensors; raises one WeightError that lists
    every missing, unexpected and wrongly shaped tensor."""
    load_state_dict(model, iter_tensors(model_dir))


def load_state_dict(model, tensors) -> None:
    params = model.named_parameters()
    head_name = f"{model.spec.head.name}.weight"
    seen, unexpected, wrong, other = set(), [], [], []
    items = tensors.items() if isinstance(tensors, dict) else tensors
    for name, t in items:
        if name in seen:
            other.append(f"tensor {name} appears twice")
            continue
        p = params.get(name)
        if p is None:
            unexpected.append(name)
            continue
        seen.add(name)
        if tuple(t.shape) != tuple(p.tensor.shape):
            wrong.append(f"{name}: checkpoint {tuple(t.shape)}, model {tuple(p.tensor.shape)}")
            continue
        if not (t.dtype.is_floating_point or t.dtype in (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8)):
            other.append(f"{name}: unsupported dtype {t.dtype}")
            continue
        if not t.dtype.is_floating_point:
            p.replace(t.to(torch.int32).to(p.tensor.device)) if p._replace else other.append(
                f"{name}: an integer tensor for a floating-point parameter")
            continue
        if p.keep_f32 and t.dtype == torch.float32 and p.tensor.dtype != torch.float32:
            p.replace(t.to(p.tensor.device))
        else:
            p.tensor.copy_(t.to(p.tensor.dtype))
    missing = [n for n in params if n not in seen]
    if head_name in missing and model.spec.head.tie_to_embedding_when_missing \
            and f"{model.spec.embed_name}.weight" in seen:
        model.tie_head_to_embedding()
        missing.remove(head_name)
    if missing or unexpected or wrong or other:
        raise WeightError(missing, unexpected, wrong, other)
