"""The generic causal language model: embedding, layers run in the order the description gives,
final norm, output head at the wanted rows.  It is built from a `ModelSpec` alone; the embedding and
the head are parts chosen by kind like the layers' (`parts/ends.py`).

Reference for the flow: csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:89-101 (model loop),
:123-127 (head); gathering the wanted rows before the head follows the generic template
csrc/layers/causal_lm_templates/text_causal_lm.hpp:59-75 rather than MiniCPM4's own class, which
computes logits at every position.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import kernels
from ..config.spec import ModelSpec, PartSpec
from ..parts import BuildContext, Param, ResidualStream, build_block
from ..parts.registry import build_embedding, build_head, build_norm


class CausalLM:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        spec.validate()
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        ctx = BuildContext(dtype=dtype, device=self.device)
        self.embedding = build_embedding(PartSpec(spec.embed_kind, dict(spec.embed_params, vocab_size=spec.vocab_size,
                                                                         hidden_size=spec.hidden_size, scale=spec.embed_scale)), ctx)
        self.blocks = [build_block(ls, ctx) for ls in spec.layers]
        self.final_norm = build_norm(spec.final_norm, ctx)
        self.output_head = build_head(PartSpec(spec.head.kind, dict(spec.head.params, vocab_size=spec.vocab_size,
                                                                    hidden_size=spec.hidden_size, scale=spec.head.scale)), ctx)
        # cache entry -> what its writer's mixer needs
        self.cache_needs: List = [None] * spec.num_cache_entries()
        for run in spec.order:
            if run.cache is not None and run.writes_cache:
                self.cache_needs[run.cache] = self.blocks[run.layer].cache_need()
        for run in spec.order:
            if run.cache is not None and not run.writes_cache:
                need = self.blocks[run.layer].cache_need()
                if need != self.cache_needs[run.cache]:
                    raise ValueError(f"layer {run.layer} reads cache entry {run.cache}, whose writer keeps "
                                     f"{self.cache_needs[run.cache]}, but needs {need}")

    # ---- tensors by checkpoint name ---------------------------------------------------------
    @property
    def embed(self) -> torch.Tensor:
        """The embedding's table."""
        return self.embedding.table

    @property
    def head(self) -> torch.Tensor:
        """The head's matrix (the embedding's table itself when the head is tied)."""
        return self.output_head.weight

    @property
    def head_is_tied(self) -> bool:
        return self.output_head.tied

    def named_parameters(self) -> Dict[str, Param]:
        out: Dict[str, Param] = {}
        for name, p in self.embedding.named_parameters().items():
            out[f"{self.spec.embed_name}.{name}"] = p
        for b in self.blocks:
            out.update(b.named_parameters())
        for name, p in self.final_norm.named_parameters().items():
            out[f"{self.spec.final_norm_name}.{name}"] = p
        for name, p in self.output_head.named_parameters().items():
            out[f"{self.spec.head.name}.{name}"] = p
        return out

    def tie_head_to_embedding(self) -> None:
        """The head reads the embedding table itself (one tensor, no copy); the embedding's scale
        is applied at lookup, so the table the head sees is the unscaled one
        (python/infinilm/modeling_utils.py:342-351)."""
        self.output_head.tie(self.embedding.table)

    def weight_bytes(self) -> int:
        seen = {}
        for p in self.named_parameters().values():
            t = p.tensor
            seen[t.untyped_storage().data_ptr() if t.device.type != "meta" else id(t)] = t.untyped_storage().nbytes()
        return sum(seen.values())

    # ---- forward ------------------------------------------------------------------------------
    def forward(self, batch, cache) -> torch.Tensor:
        """float32 logits [len(batch.want_rows), vocab] for the tokens of `batch`."""
        stream = ResidualStream(self.embedding.forward(batch.token_ids))
        taps = batch.taps
        if taps is not None:
            taps["embed"] = stream.residual.clone()
        for i, run in enumerate(self.spec.order):
            view = cache.view(run.cache, batch, run.writes_cache) if run.cache is not None else None
            self.blocks[run.layer].forward(stream, batch, view)
            if taps is not None:
                taps[f"run{i}"] = (stream.residual.clone(), None if stream.pending is None else stream.pending.clone(),
                                   stream.pending_scale)
        if batch.num_wanted == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if not batch.wants_all_rows:
            last = ResidualStream(kernels.gather_rows(stream.residual, batch.want_rows))
            if stream.pending is not None:
                pend = stream.pending
                if pend.dim() == 3:   # parts of a K-split product: the rows of every part
                    pend = torch.stack([kernels.gather_rows(p, batch.want_rows) for p in pend])
                else:
                    pend = kernels.gather_rows(pend, batch.want_rows)
                last.push(pend, stream.pending_scale)
            stream = last
        x = self.final_norm.forward(stream)
        return self.output_head.forward(x)
