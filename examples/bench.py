"""End-to-end generation speed through the engine loop (scheduler, step function, sampler), over
a grid of batch sizes and input/output lengths ordered by the cache they need, in the manner of
the reference's examples/bench.py (case grid :100-160, one timed generate per case :592-700).

    python examples/bench.py --model DIR [--skip-load] --batch-size 1,8 --input-len 128,2048
        --output-len 64 [--dtype bfloat16] [--enable-graph] [--block-size 64] [--warmup]
    python examples/bench.py --shape 0.5b --batch-size 64 --prompt-len-range 128,2048 --output-len 128 ...

`--shape 8b|0.5b|2b` stands for --model with --skip-load: one of the benchmark shapes of
examples/shapes.py with random weights.  Prompts are random token ids (no tokenizer is needed) of
the asked length, or, with `--prompt-len-range LO,HI`, of lengths drawn uniformly from [LO, HI]
with the case's seed, one length a request (a mixed load: portions of long prompts run beside the
decoded tokens of short ones); every request generates exactly --output-len tokens (ignore_eos).
For each case one line: time to first token (all prompts admitted together, portions under the
token budget), prefill, decode and total tokens a second, the distribution of the step times (all
steps, and the steps after the last prompt was done), and the host's share of the decode steps.
"""
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import torch  # noqa: E402

from infinilm_amd import LLM, SamplingParams  # noqa: E402
from infinilm_amd.base_config import BaseConfig  # noqa: E402


def int_list(text) -> list:
    return [int(x) for x in str(text).replace("[", "").replace("]", "").split(",") if x.strip()]


def test_cases(cfg_json: dict, batch_sizes, input_lens, output_lens):
    """Cases in ascending order of the bytes of cache they fill (bfloat16 keys and values)."""
    heads = cfg_json["num_attention_heads"]
    d = cfg_json.get("head_dim") or cfg_json["hidden_size"] // heads
    nkv = cfg_json.get("num_key_value_heads") or heads
    layers = cfg_json["num_hidden_layers"]
    cases = []
    for b in batch_sizes:
        for i in input_lens:
            for o in output_lens:
                nbytes = 2 * 2 * b * (i + o) * nkv * d * layers
                cases.append((nbytes, {"batch_size": b, "input_len": i, "output_len": o,
                                       "kvcache_gb": round(nbytes / 2 ** 30, 3)}))
    return [c for _, c in sorted(cases, key=lambda nc: nc[0])]


def percentiles(ms: list) -> dict:
    """p50 / p90 / p99 / max of a list of milliseconds (nearest rank)."""
    if not ms:
        return {}
    v = sorted(ms)
    at = lambda q: round(v[min(len(v) - 1, int(q * len(v)))], 3)
    return {"n": len(v), "p50": at(0.50), "p90": at(0.90), "p99": at(0.99), "max": round(v[-1], 3)}


def run_case(llm: LLM, case: dict, seed: int, sp_kwargs: dict) -> dict:
    b, n_in, n_out = case["batch_size"], case["input_len"], case["output_len"]
    V = llm.model.spec.vocab_size
    gen = torch.Generator().manual_seed(seed)
    lo, hi = case.get("prompt_len_range") or (n_in, n_in)
    lens = torch.randint(lo, hi + 1, (b,), generator=gen).tolist()
    prompts = [torch.randint(0, V, (n,), generator=gen).tolist() for n in lens]
    sp = SamplingParams(max_tokens=n_out, ignore_eos=True, **sp_kwargs)
    eng = llm.engine
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reqs = [eng.add_request(p, sp.clone()) for p in prompts]
    first = {}
    steps = 0
    t_first_all = None
    step_ms = []
    last = t0
    while any(not r.is_finished() for r in reqs):
        eng.step()   # the sampled tokens come back to the host inside: the step is complete here
        steps += 1
        now = time.perf_counter()
        step_ms.append(1e3 * (now - last))
        last = now
        for r in reqs:
            if r.request_id not in first and r.get_num_generated_tokens() > 0:
                first[r.request_id] = now - t0
        if t_first_all is None and len(first) == len(reqs):
            t_first_all = now
            steps_at_first = steps
            mid = eng.stats()
    t1 = time.perf_counter()
    after = eng.stats()
    failed = [r.error for r in reqs if r.error]
    if failed:
        return dict(case, error=failed[0])
    ttft = sum(first.values()) / len(first)
    prefill_s = t_first_all - t0
    decode_s = t1 - t_first_all
    decode_tokens = sum(r.get_num_generated_tokens() for r in reqs) - b
    generated = sum(r.get_num_generated_tokens() for r in reqs)
    return dict(case,
                prompt_tokens=sum(lens),
                ttft_ms=round(1e3 * ttft, 2),
                prefill_tok_s=round(sum(lens) / prefill_s, 1),
                total_tok_s=round((sum(lens) + generated) / (t1 - t0), 1),
                output_tok_s=round(generated / (t1 - t0), 1),
                step_ms=percentiles(step_ms),
                decode_step_ms=percentiles(step_ms[steps_at_first:]),
                decode_tok_s=round(decode_tokens / decode_s, 1) if decode_tokens > 0 and decode_s > 0 else None,
                decode_ms_per_step=round(1e3 * decode_s / max(steps - steps_at_first, 1), 3),
                total_ms=round(1e3 * (t1 - t0), 2),
                # host milliseconds of a decode step: scheduling, building and launching the step,
                # bookkeeping (the wait for the device is inside the sampler's copy of the tokens: not counted)
                decode_host_ms_per_step=round(1e3 * sum(after[k] - mid[k] for k in ("schedule_s", "step_s", "update_s"))
                                              / max(steps - steps_at_first, 1), 3))


def main(argv=None) -> int:
    import argparse
    extra = argparse.ArgumentParser(add_help=False)
    extra.add_argument("--shape", choices=["8b", "0.5b", "2b"], default=None)
    extra.add_argument("--layers", type=int, default=0, help="with --shape: run this many layers instead of the shape's")
    extra.add_argument("--prompt-len-range", type=str, default=None, help="LO,HI: a length of its own for every request")
    ex, rest = extra.parse_known_args(sys.argv[1:] if argv is None else argv)
    if ex.shape:
        rest = ["--model", f"shape:{ex.shape}", "--skip-load"] + rest
    cfg = BaseConfig(rest, batch_size_type=str)
    if ex.shape:
        from shapes import shape_config
        model_path = cfg_json = shape_config(ex.shape, ex.layers)
    else:
        model_path = os.path.expanduser(cfg.model)
        with open(os.path.join(model_path, "config.json")) as f:
            cfg_json = json.load(f)
    input_lens = int_list(cfg.input_len)
    len_range = None
    if ex.prompt_len_range:
        len_range = tuple(int_list(ex.prompt_len_range))
        if len(len_range) != 2 or not 1 <= len_range[0] <= len_range[1]:
            raise SystemExit("--prompt-len-range takes LO,HI with 1 <= LO <= HI")
        input_lens = [len_range[1]]   # the cache is sized for the longest
    cases = test_cases(cfg_json, int_list(cfg.batch_size), input_lens, int_list(cfg.output_len))
    if len_range:
        cases = [dict(c, prompt_len_range=list(len_range)) for c in cases]
    page = cfg.block_size
    need = max(c["batch_size"] * (-(-(c["input_len"] + c["output_len"]) // page) + 1) for c in cases)
    llm = LLM(model_path=model_path, dtype=cfg.dtype, max_batch_size=max(c["batch_size"] for c in cases),
              num_blocks=max(need, 1), block_size=page, enable_graph=cfg.enable_graph,
              skip_load=cfg.skip_load or cfg.random_weights, max_num_batched_tokens=cfg.max_num_batched_tokens,
              chunk_size=cfg.chunk_size, admission=cfg.admission, seed=cfg.seed,
              enable_prefix_caching=cfg.enable_prefix_caching, look_ahead=cfg.look_ahead,
              record_graphs_at_start=cfg.record_graphs_at_start)
    sp_kwargs = dict(temperature=cfg.temperature, top_k=cfg.top_k, top_p=cfg.top_p)
    try:
        if cfg.warmup:
            print("=================== warmup start ===================", flush=True)
            # with graphs a step's shape is recorded the second time it comes: the warm-up runs each case twice, so that
            # the prompts' steps of the measured run are replays and not recordings
            # (prompts of its own for each pass: with prefix caching a prompt that comes again is not computed again)
            for rep in range(2 if cfg.enable_graph else 1):
                for c in cases:
                    run_case(llm, dict(c, output_len=min(c["output_len"], 4)), cfg.seed + 500 * rep, sp_kwargs)
            print("=================== warmup done ====================", flush=True)
        for i, c in enumerate(cases):   # prompts of their own for every case: no case finds another's pages
            print(json.dumps(run_case(llm, c, cfg.seed + 1 + 1000 * (i + 1), sp_kwargs)), flush=True)
    finally:
        llm.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
