"""From a model folder to a built model with its weights, and to a step runner with a cache."""
from __future__ import annotations

import warnings
from typing import Optional

import torch

from ..cache import CacheManager
from ..config.registry import load_model_config
from ..weights.loader import load_weights
from .model import CausalLM
from .step import StepRunner

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "fp32": torch.float32, "bf16": torch.bfloat16,
           torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def resolve_dtype(dtype, config_dtype: Optional[str]) -> torch.dtype:
    """`dtype` given wins; else config.json's `dtype`/`torch_dtype` (csrc/config/model_config.cpp:28-39).
    float16 (a dtype of its own in the reference, csrc/utils.hpp:150-167) runs in bfloat16 here, with
    a warning: the kernels take float32 and bfloat16, and bfloat16 keeps float16's range-safe
    accumulation in float32 but three bits less of mantissa in weights, activations and cache."""
    if dtype is None:
        if config_dtype is None:
            raise ValueError("No dtype or torch_dtype found in config, and none was given")
        dtype = config_dtype
    if dtype in ("float16", "fp16", "half", torch.float16):
        warnings.warn("infinilm_amd: float16 was asked for; this engine computes in bfloat16 instead "
                      "(same range as float32, 8 instead of 11 bits of precision): results differ from a "
                      "float16 run by rounding. Pass dtype='float32' for the exact path.", RuntimeWarning, stacklevel=2)
        dtype = "bfloat16"
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"Unsupported dtype string: {dtype}") from None


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("infinilm_amd runs on an AMD GPU only (device 'cuda:N' under ROCm); "
                           "there is no CPU path")
    return device


def build_model(model_dir_or_config, dtype=None, device="cuda:0") -> CausalLM:
    """The model for a config.json (a folder or its parsed dict), parameters uninitialised."""
    arch, cfg = load_model_config(model_dir_or_config)
    spec = arch.build_spec(cfg)
    dt = resolve_dtype(dtype, getattr(cfg, "dtype", None))
    model = CausalLM(spec, dt, device)
    model.config = cfg
    return model


def load_model(model_dir: str, dtype=None, device="cuda:0") -> CausalLM:
    device = require_gpu(device)
    from ..csrc import lib
    lib.load()  # compile the kernels first if need be, and fail early without them
    model = build_model(model_dir, dtype, device)
    load_weights(model, model_dir)
    return model


def fragment_copy_bytes(model: CausalLM) -> int:
    """Bytes the projections' second copies in fragment order take once every product has packed its own: they are
    made at a product's first use with 17 or more rows (`FusedLinear.frag_weight`), long after the cache pool has
    been sized, so the pool leaves room for them."""
    from .. import kernels
    from ..parts.linear import FusedLinear
    total, seen, stack = 0, set(), [model]
    while stack:
        o = stack.pop()
        if id(o) in seen:
            continue
        seen.add(id(o))
        if isinstance(o, FusedLinear):
            if kernels.frag_weight_ok(o.weight):
                total += o.weight.numel() * o.weight.element_size()
        elif isinstance(o, (list, tuple)):
            stack.extend(o)
        elif isinstance(o, dict):
            stack.extend(o.values())
        elif type(o).__module__.startswith("infinilm_amd") and hasattr(o, "__dict__"):
            stack.extend(vars(o).values())
    return total


def pages_that_fit(model: CausalLM, page_size: int, memory_fraction: float = 0.9, reserve_bytes: int = 4 << 30) -> int:
    """Pages per group that `memory_fraction` of the device's free memory holds (after `reserve_bytes`
    for activations, graphs and workspaces, and after the weights' copies in fragment order that are still to
    be made), for `num_pages=None`: the cache takes what the weights leave, on a 288 GB part some hundred
    thousand tokens for a model of this size."""
    from ..cache.needs import PagedKV
    reserve_bytes += fragment_copy_bytes(model)
    elem = torch.empty((), dtype=model.dtype).element_size()
    per_page = sum(2 * n.num_kv_heads * n.head_dim * page_size * elem for n in model.cache_needs if isinstance(n, PagedKV))
    if per_page == 0:
        return 1
    free, _ = torch.cuda.mem_get_info(model.device)
    usable = int(free * memory_fraction) - reserve_bytes
    if usable < per_page:
        raise RuntimeError(f"no room for a cache: {free / 2**30:.1f} GiB free on {model.device}, a page of every layer "
                           f"takes {per_page / 2**20:.1f} MiB")
    return usable // per_page


def make_runner(model: CausalLM, num_pages: Optional[int], page_size: int, max_requests: int,
                enable_graph: bool = False, prefix_caching: bool = False) -> StepRunner:
    """`num_pages=None`: as many pages as fit into the free device memory (see `pages_that_fit`).
    `prefix_caching`: whole pages of computed tokens are published for later requests with the same
    beginning (where the model's cache entries allow it: `runner.cache.prefix_caching` tells)."""
    if num_pages is None:
        num_pages = pages_that_fit(model, page_size)
    cache = CacheManager(model.cache_needs, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=model.dtype, device=model.device, prefix_caching=prefix_caching)
    return StepRunner(model, cache, enable_graph=enable_graph)
