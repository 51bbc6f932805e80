"""Command-line options with the reference's names and meanings
(python/infinilm/base_config.py:182-480), restricted to what a single-GPU engine for one
architecture has.  Options of the reference that do not apply here (several GPUs, quantization,
other backends, servers, images) are not offered."""
from __future__ import annotations

import argparse
from typing import List, Optional


class BaseConfig:
    def __init__(self, argv: Optional[List[str]] = None, batch_size_type=int):
        """`batch_size_type=str` lets a benchmark take a list ("1,8,64") where generation takes a number."""
        ap = argparse.ArgumentParser(description="infinilm_amd generation example")
        ap.add_argument("--model", type=str, required=True, help="model directory (config.json + safetensors)")
        ap.add_argument("--device", type=str, default="auto", help="always the AMD GPU; kept for compatibility")
        ap.add_argument("--device-id", type=int, default=0)
        ap.add_argument("--dtype", type=str, default=None, choices=["float32", "bfloat16", "float16"],
                        help="overrides config.json's dtype; float32 is true 32-bit throughout; float16 is run "
                             "as bfloat16, with a warning")
        ap.add_argument("--batch-size", type=batch_size_type, default=batch_size_type(1),
                        help="number of copies of the prompt")
        ap.add_argument("--prompt", type=str, default="How are you")
        ap.add_argument("--prompt-ids", type=str, default=None,
                        help="comma-separated token ids instead of --prompt (no tokenizer needed)")
        ap.add_argument("--max-new-tokens", type=int, default=512)
        ap.add_argument("--top-k", type=int, default=1)
        ap.add_argument("--top-p", type=float, default=1.0)
        ap.add_argument("--temperature", type=float, default=1.0)
        ap.add_argument("--enable-paged-attn", action="store_true", help="accepted; the cache is always paged")
        ap.add_argument("--attn", type=str, default="default", choices=["default", "paged-attn"])
        ap.add_argument("--num-blocks", type=int, default=512, help="pages of the cache pool; 0: what the free device memory holds")
        ap.add_argument("--block-size", type=int, default=256)
        ap.add_argument("--max-batch-size", type=int, default=8)
        ap.add_argument("--max-num-batched-tokens", type=int, default=None)
        ap.add_argument("--chunk-size", type=int, default=None, help="longest portion of a prompt in one step")
        ap.add_argument("--admission", type=str, default="optimistic", choices=["optimistic", "reserve_full"])
        ap.add_argument("--enable-graph", action="store_true")
        ap.add_argument("--record-graphs-at-start", action="store_true",
                        help="with --enable-graph: record every decode step size before the first request")
        ap.add_argument("--disable-look-ahead", dest="look_ahead", action="store_false", default=None,
                        help="with --enable-graph: wait for a step's tokens before the next step is launched")
        ap.add_argument("--disable-prefix-caching", dest="enable_prefix_caching", action="store_false", default=True,
                        help="do not reuse the cached pages of an earlier request with the same beginning")
        ap.add_argument("--skip-load", action="store_true", help="draw random weights instead of loading")
        ap.add_argument("--random-weights", action="store_true", help="same as --skip-load")
        ap.add_argument("--seed", type=int, default=0)
        ap.add_argument("--ignore-eos", action="store_true")
        ap.add_argument("--warmup", action="store_true")
        ap.add_argument("--verbose", action="store_true")
        ap.add_argument("--log-level", type=str, default="INFO")
        ap.add_argument("--input-len", type=str, default="10")
        ap.add_argument("--output-len", type=str, default="20")
        args = ap.parse_args(argv)
        for k, v in vars(args).items():
            setattr(self, k, v)

    @staticmethod
    def get_device_str(device: str, device_id: int = 0) -> str:
        return f"cuda:{device_id}"
