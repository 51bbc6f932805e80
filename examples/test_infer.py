"""Generates for one prompt copied --batch-size times and prints the responses, like the
reference's examples/test_infer.py.

    python examples/test_infer.py --model DIR [--dtype bfloat16] [--batch-size 4]
        [--prompt "How are you" | --prompt-ids 1,5,9] [--max-new-tokens 64]
        [--top-k 1 --top-p 1.0 --temperature 1.0] [--num-blocks 512 --block-size 256]
        [--disable-prefix-caching]
"""
import logging
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from infinilm_amd import LLM, SamplingParams  # noqa: E402
from infinilm_amd.base_config import BaseConfig  # noqa: E402


def main(argv=None) -> int:
    cfg = BaseConfig(argv)
    logging.basicConfig(level=getattr(logging, cfg.log_level.upper(), logging.INFO))
    model = LLM(model_path=os.path.expanduser(cfg.model), device=cfg.get_device_str(cfg.device, cfg.device_id),
                dtype=cfg.dtype, max_batch_size=max(cfg.batch_size, 1), max_tokens=cfg.max_new_tokens,
                num_blocks=cfg.num_blocks or None, block_size=cfg.block_size, temperature=cfg.temperature, top_k=cfg.top_k,
                top_p=cfg.top_p, enable_graph=cfg.enable_graph, attn_backend=cfg.attn,
                skip_load=cfg.skip_load or cfg.random_weights, max_num_batched_tokens=cfg.max_num_batched_tokens,
                chunk_size=cfg.chunk_size, admission=cfg.admission, seed=cfg.seed,
                enable_prefix_caching=cfg.enable_prefix_caching, look_ahead=cfg.look_ahead,
                record_graphs_at_start=cfg.record_graphs_at_start)
    sp = SamplingParams(temperature=cfg.temperature, top_p=cfg.top_p, top_k=cfg.top_k, max_tokens=cfg.max_new_tokens,
                        ignore_eos=cfg.ignore_eos)
    t1 = time.time()
    print("=================== start generate ====================")
    try:
        if cfg.prompt_ids is not None:
            ids = [int(x) for x in cfg.prompt_ids.split(",") if x.strip()]
            outputs = model.generate(prompt_token_ids=[ids] * cfg.batch_size, sampling_params=sp)
        elif model.tokenizer is not None and getattr(model.tokenizer, "chat_template", None):
            conversations = [[{"role": "user", "content": cfg.prompt}] for _ in range(cfg.batch_size)]
            outputs = model.chat(conversations, sampling_params=sp)
        else:
            outputs = model.generate([cfg.prompt] * cfg.batch_size, sampling_params=sp)
    finally:
        model.close()
    t2 = time.time()
    for i, output in enumerate(outputs):
        print(f"Request {i}:")
        print("===Query===")
        print(output.prompt if output.prompt is not None else output.prompt_token_ids)
        print("===Response===")
        print(output.outputs[0].text if output.outputs[0].text else output.outputs[0].token_ids)
        print("")
    print(f"total_time: {round((t2 - t1) * 1000, 2)} ms")
    return 0


if __name__ == "__main__":
    sys.exit(main())
