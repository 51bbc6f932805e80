"""Decode and prefill throughput of the engine at MiniCPM4-8B size with random weights on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers L]

A "step" is one decode step of the engine's own step function followed by greedy sampling, with
`--batch` requests that each hold `--context` tokens in the paged cache when the last timed step
ends.  One JSON line is printed: `value` is decoded tokens a second at the default batch;
`prefill` is one 2,048-token prompt in one step (the median of seven passes timed with events);
`roofline` prices the decode step against HBM bandwidth (every weight it uses read once, plus the
cache of the live requests); `points` holds decode at batch 1, 32 and 64 and `points_frac` the same
pricing of each; `fp32` the batch-8 step and the prefill on the true 32-bit path.  Peaks are MI355X's
published ones (HBM 8 TB/s; dense MFMA bf16 2.5 PFLOP/s, fp32 157.3 TFLOP/s).  Weights are random (N(0, 0.02), norms 1 + N(0, 0.02)) and the
cache of the context is filled with random keys and values instead of being computed: the timed
steps do all of their work.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def config_8b(layers: int) -> dict:
    """The layer sizes of the MiniCPM4-8B shape."""
    sys.path.insert(0, os.path.join(ROOT, "examples"))
    from shapes import shape_config
    return shape_config("8b", layers)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=32, help="layers to run (the 8B configuration has 32)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel of a decode step eagerly")
    ap.add_argument("--prefill-only", action="store_true", help="only the prefill measurement (for profiling)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 32 / 64 points, the prefill and the 32-bit record")
    ap.add_argument("--no-fp32", action="store_true", help="skip the 32-bit record (bfloat16 runs only)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this engine has no multi-GPU path (N>1 is not run)")
        return 2

    import torch
    from infinilm_amd.csrc import lib
    from infinilm_amd.engine.loading import require_gpu

    require_gpu("cuda:0")
    lib.load()
    FULL_LAYERS = 32
    cfg = config_8b(args.layers)
    record = measure(args, cfg, args.dtype, FULL_LAYERS, full=True)
    if args.dtype == "bfloat16" and not args.no_points and not args.no_fp32 and not args.prefill_only:
        torch.cuda.empty_cache()
        f = measure(args, cfg, "float32", FULL_LAYERS, full=False)
        record["fp32"] = {"decode_b%d" % args.batch: f["value"], "ms_per_step": f["ms_per_step"], "hbm_frac": f["roofline"]["frac"],
                          "prefill_ms": f["prefill"]["ms"], "prefill_frac": f["prefill"]["frac"]}
    print(json.dumps(record))
    return 0


def measure(args, cfg, dtype, FULL_LAYERS, full):
    """One dtype's record; `full`: with the batch 1 / 32 / 64 points."""
    import torch
    from infinilm_amd.engine.loading import build_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    from infinilm_amd.sampling import Sampler, SamplingParams
    from infinilm_amd.weights import fill_random_

    model = build_model(cfg, dtype, "cuda:0")
    fill_random_(model, seed=0, std=0.02, norm_init="one_plus")
    torch.cuda.synchronize()
    spec = model.spec
    H, V, L = spec.hidden_size, spec.vocab_size, len(spec.order)
    esize = 2 if dtype == "bfloat16" else 4
    dkey = "bf16" if dtype == "bfloat16" else "fp32"

    max_b = max(args.batch, 1 if (args.no_points or not full) else 64)
    ps = args.page_size
    pages_per_req = -(-(args.context + 1) // ps)
    num_pages = max(max_b * pages_per_req, -(-args.prefill_tokens // ps)) + 4
    runner = make_runner(model, num_pages=num_pages, page_size=ps, max_requests=max_b + 1,
                         enable_graph=not args.no_graph)
    cache = runner.cache
    for e in cache.k:
        cache.k[e].normal_(0, 1.0)
        cache.v[e].normal_(0, 1.0)
    sampler = Sampler(0)
    greedy = SamplingParams(top_k=1)
    gen = torch.Generator().manual_seed(7)

    # every tensor but the embedding table and the head: what the layers and the final norm read once a step
    outer = {model.embed.data_ptr(), model.head.data_ptr()}
    inner = [p.tensor for p in model.named_parameters().values() if p.tensor.data_ptr() not in outer]
    layer_weight_bytes = sum(t.numel() * t.element_size() for t in inner)
    head_bytes = model.head.numel() * model.head.element_size()

    def decode(batch: int, steps: int, warmup: int):
        ids = [f"d{batch}_{i}" for i in range(batch)]
        start = args.context - (steps + warmup)
        assert start > 0
        for rid in ids:
            cache.admit(rid)
            cache.reserve(rid, start)
            cache.commit(rid, start)   # the context's keys and values are the random fill
        toks = torch.randint(0, V, (batch,), generator=gen).tolist()

        def one(toks):
            logits = runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, toks)])
            return sampler.sample(logits, [(greedy, i, 0) for i in range(batch)])

        for _ in range(warmup):
            toks = one(toks)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            toks = one(toks)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx_mean = args.context - steps / 2.0
        for rid in ids:
            cache.release(rid)
        ms = dt / steps * 1e3
        kv_bytes = batch * ctx_mean * cache.bytes_per_token()
        step_bytes = layer_weight_bytes + head_bytes + batch * H * esize + kv_bytes
        return {"tok_s": batch * steps / dt, "ms": ms, "bytes": step_bytes, "gbs": step_bytes / (dt / steps) / 1e9}

    def prefill():
        # one prompt of T tokens in one step, logits at its last place
        T = args.prefill_tokens
        prompt = torch.randint(0, V, (T,), generator=gen).tolist()
        times = []
        passes = 7 if dtype == "bfloat16" else 3
        for i in range(passes + 1):   # the first pass warms up (the library chooses its kernels there)
            rid = f"p{i}"
            cache.admit(rid)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            logits = runner.step([StepEntry(rid, prompt, [T - 1])])
            sampler.sample(logits, [(greedy, 0, 0)])
            e1.record()
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3)
            cache.release(rid)
        pt = sorted(times[1:])[len(times[1:]) // 2]   # the median
        mat_params = sum(t.numel() for t in inner if t.dim() == 2)
        flops = 2.0 * T * mat_params + 4.0 * T * T / 2.0 * cfg["num_attention_heads"] * cfg["head_dim"] * L + 2.0 * V * H
        return {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3), "frac": round(flops / pt / FLOP_PEAK[dkey], 4)}

    if args.prefill_only:
        return {"prefill": prefill()}
    main_pt = decode(args.batch, args.steps, args.warmup)
    record = {
        "metric": "decode tokens/s, MiniCPM4-8B shape, batch %d, context %d" % (args.batch, args.context),
        "value": round(main_pt["tok_s"], 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(main_pt["ms"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic: random weights, random token ids, random-filled cache",
        "config": {"model": "MiniCPM4-8B shape (random weights)", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single-gpu", "num_hidden_layers": FULL_LAYERS, "layers_run": L, "hidden_size": H,
                   "num_attention_heads": 32, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 16384,
                   "vocab_size": V, "rope": "longrope, 64 factors", "tied_head": False, "page_size": ps,
                   "prefill_tokens": args.prefill_tokens},
        "roofline": {"bound": "hbm", "achieved": round(main_pt["gbs"], 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(main_pt["gbs"] * 1e9 / HBM_PEAK, 4)},
    }
    if not args.no_points:
        k = max(8, args.steps // 2)
        if full:
            pts = {b: decode(b, k, args.warmup) for b in (1, 32, 64)}
            record["points"] = {f"decode_b{b}": round(p["tok_s"], 2) for b, p in pts.items()}
            # the same pricing as `roofline` for each point: bytes the step has to read / its time / the HBM peak
            record["points_frac"] = {f"decode_b{b}": round(p["gbs"] * 1e9 / HBM_PEAK, 4) for b, p in pts.items()}
        record["prefill"] = prefill()
    del runner, cache, model
    return record


if __name__ == "__main__":
    sys.exit(main())
