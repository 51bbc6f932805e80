"""End-to-end generation speed through the engine loop (scheduler, step function, sampler), over
a grid of batch sizes and input/output lengths ordered by the cache they need, in the manner of
the reference's examples/bench.py (case grid :100-160, one timed generate per case :592-700).

    python examples/bench.py --model DIR [--skip-load] --batch-size 1,8 --input-len 128,2048
        --output-len 64 [--dtype bfloat16] [--enable-graph] [--block-size 64] [--warmup]

Prompts are random token ids of the asked length (no tokenizer is needed); every request
generates exactly --output-len tokens (ignore_eos).  For each case one line:
time to first token (all prompts admitted together, portions under the token budget), prefill
and decode tokens a second, and the host's share of the decode steps.
"""
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

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


def run_case(llm: LLM, case: dict, seed: int, sp_kwargs: dict) -> dict:
    b, n_in, n_out = case["batch_size"], case["input_len"], case["output_len"]
    V = llm.model.spec.vocab_size
    gen = torch.Generator().manual_seed(seed)
    prompts = [torch.randint(0, V, (n_in,), generator=gen).tolist() for _ in range(b)]
    sp = SamplingParams(max_tokens=n_out, ignore_eos=True, **sp_kwargs)
    eng = llm.engine
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reqs = [eng.add_request(p, sp.clone()) for p in prompts]
    first = {}
    steps = 0
    t_first_all = None
    while any(not r.is_finished() for r in reqs):
        eng.step()   # the sampled tokens come back to the host inside: the step is complete here
        steps += 1
        now = time.perf_counter()
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
    return dict(case,
                ttft_ms=round(1e3 * ttft, 2),
                prefill_tok_s=round(b * n_in / prefill_s, 1),
                decode_tok_s=round(decode_tokens / decode_s, 1) if decode_tokens > 0 and decode_s > 0 else None,
                decode_ms_per_step=round(1e3 * decode_s / max(steps - steps_at_first, 1), 3),
                total_ms=round(1e3 * (t1 - t0), 2),
                # host milliseconds of a decode step: scheduling, building and launching the step,
                # bookkeeping (the wait for the device is inside the sampler's copy of the tokens: not counted)
                decode_host_ms_per_step=round(1e3 * sum(after[k] - mid[k] for k in ("schedule_s", "step_s", "update_s"))
                                              / max(steps - steps_at_first, 1), 3))


def main(argv=None) -> int:
    cfg = BaseConfig(argv, batch_size_type=str)
    model_path = os.path.expanduser(cfg.model)
    with open(os.path.join(model_path, "config.json")) as f:
        cfg_json = json.load(f)
    cases = test_cases(cfg_json, int_list(cfg.batch_size), int_list(cfg.input_len), int_list(cfg.output_len))
    page = cfg.block_size
    need = max(c["batch_size"] * (-(-(c["input_len"] + c["output_len"]) // page) + 1) for c in cases)
    llm = LLM(model_path=model_path, dtype=cfg.dtype, max_batch_size=max(c["batch_size"] for c in cases),
              num_blocks=max(need, 1), block_size=page, enable_graph=cfg.enable_graph,
              skip_load=cfg.skip_load or cfg.random_weights, max_num_batched_tokens=cfg.max_num_batched_tokens,
              chunk_size=cfg.chunk_size, admission=cfg.admission, seed=cfg.seed,
              enable_prefix_caching=cfg.enable_prefix_caching, look_ahead=cfg.look_ahead)
    sp_kwargs = dict(temperature=cfg.temperature, top_k=cfg.top_k, top_p=cfg.top_p)
    try:
        if cfg.warmup:
            print("=================== warmup start ===================", flush=True)
            for c in cases:   # also records the HIP graphs of each batch size
                run_case(llm, dict(c, output_len=min(c["output_len"], 4)), cfg.seed, sp_kwargs)
            print("=================== warmup done ====================", flush=True)
        for i, c in enumerate(cases):   # prompts of their own for every case: no case finds another's pages
            print(json.dumps(run_case(llm, c, cfg.seed + 1 + 1000 * (i + 1), sp_kwargs)), flush=True)
    finally:
        llm.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
