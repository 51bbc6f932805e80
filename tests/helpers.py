"""Shared by the GPU tests: model folders with random weights, the plain oracle's logits, and a
small driver that feeds steps to the engine's own step function and keeps logits by (request,
position)."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

import plain_minicpm4 as P

CONFIGS = {"A": P.tiny_config_a, "B": P.tiny_config_b, "C": P.tiny_config_c, "D": P.tiny_config_d, "E": P.tiny_config_e}


def make_model_dir(path: str, cfg: dict, seed: int, store: str = "float32", sharp: bool = True):
    """Writes config.json + model.safetensors; returns the weights as the oracle should see them
    (float32 values; rounded to bfloat16 first when the file stores bfloat16)."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    W = P.plain_random_weights(cfg, seed, sharp=sharp)
    if store == "bfloat16":
        W = {k: v.to(torch.bfloat16) for k, v in W.items()}
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(dict(cfg, torch_dtype=store), fh)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"),
              metadata={"format": "pt"})
    return {k: v.to(torch.float32) for k, v in W.items()}


def random_tokens(cfg: dict, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got = got.detach().to(torch.float64).cpu()
    want = want.detach().to(torch.float64).cpu()
    return float((got - want).abs().max() / max(1.0, float(want.abs().max())))


# tolerances: measured errors are several times below these; they are never widened to pass
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


class Driver:
    """Feeds steps to a StepRunner and files the returned logits under (request, position)."""

    def __init__(self, model_dir: str, dtype: str, num_pages: int, page_size: int, max_requests: int = 8):
        from infinilm_amd.engine.loading import load_model, make_runner

        self.model = load_model(model_dir, dtype, "cuda:0")
        self.runner = make_runner(self.model, num_pages=num_pages, page_size=page_size, max_requests=max_requests)
        self.logits: Dict[Tuple[object, int], torch.Tensor] = {}

    def step(self, entries: Sequence[Tuple[object, Sequence[int]]], want_all: bool = True, end: Sequence = ()):
        from infinilm_amd.engine.step import StepEntry

        es = []
        for rid, toks in entries:
            if not self.runner.cache.has(rid):
                self.runner.cache.admit(rid)
            es.append(StepEntry(rid, list(toks), list(range(len(toks))) if want_all else []))
        starts = [self.runner.cache.length(rid) for rid, _ in entries]
        out = self.runner.step(es).cpu()
        row = 0
        if want_all:
            for (rid, toks), s in zip(entries, starts):
                for i in range(len(toks)):
                    self.logits[(rid, s + i)] = out[row]
                    row += 1
        for rid in end:
            self.runner.cache.release(rid)
        self.runner.cache.check()

    def request_logits(self, rid, n: int) -> torch.Tensor:
        return torch.stack([self.logits[(rid, i)] for i in range(n)])
