"""The Python entry point, in the manner of the reference's `infinilm.LLM`
(python/infinilm/llm/llm.py:335-559) with `EngineConfig`'s names and meanings
(python/infinilm/config/engine_config.py:42-93)."""
from __future__ import annotations

import os
from typing import List, Optional, Sequence, Union

import torch

from .engine.llm_engine import LLMEngine
from .engine.loading import build_model, load_model, make_runner, require_gpu
from .engine.request import RequestOutput
from .sampling import SamplingParams


def _load_tokenizer(model_path: str):
    names = ("tokenizer.json", "tokenizer.model", "tokenizer_config.json")
    if not any(os.path.isfile(os.path.join(model_path, n)) for n in names):
        return None
    try:
        from transformers import AutoTokenizer  # a tokenizer only; no model code is taken from there
        return AutoTokenizer.from_pretrained(model_path, trust_remote_code=True)
    except Exception as exc:  # noqa: BLE001
        import warnings
        warnings.warn(f"tokenizer files found in {model_path} but loading failed ({exc}); pass token ids instead")
        return None


class LLM:
    """Offline generation.

    model_path      folder with config.json and safetensors (or, with `random_weights=True`, a
                    folder with config.json only, or a config dict: weights are drawn from `seed`)
    dtype           "bfloat16" | "float32" | None (config.json's); float32 is true 32-bit throughout
    max_batch_size  most requests in flight
    max_tokens      default cap of generated tokens per request
    num_blocks / block_size   pages of the cache pool (None: what the free device memory holds) / tokens a page
    temperature / top_p / top_k   defaults of requests that bring no SamplingParams
    max_num_batched_tokens / chunk_size   token budget of a step / longest portion of a prompt
    admission       "optimistic" (preempt when pages run out) | "reserve_full" (the reference's check)
    look_ahead      with enable_graph: a decode step is launched before the tokens of the one before it are
                    back on the host (None: on whenever enable_graph is)
    record_graphs_at_start   with enable_graph: every decode step size that max_batch_size requests within the
                    model's positions and the pool's pages can need is recorded before the first request (the
                    reference records when the engine is built); otherwise a size is recorded the second time it comes
    enable_prefix_caching   whole pages of computed tokens stay findable for later requests that begin
                    with the same tokens (the reference's default; off where a model's cache entries
                    keep a window or a state of their own)
    """

    def __init__(self, model_path, device: str = "cuda", dtype: Optional[str] = None, cache_type: str = "paged",
                 max_batch_size: int = 16, max_tokens: int = 4096, num_blocks: Optional[int] = 512, block_size: int = 256,
                 max_cache_len: Optional[int] = None, temperature: float = 1.0, top_p: float = 0.8, top_k: int = 1,
                 enable_graph: bool = False, attn_backend: str = "default", skip_load: bool = False,
                 enable_prefix_caching: bool = True, max_num_batched_tokens: Optional[int] = None,
                 chunk_size: Optional[int] = None, admission: str = "optimistic", seed: int = 0,
                 random_weights: bool = False, random_std: float = 0.02, tokenizer=None,
                 look_ahead: Optional[bool] = None, record_graphs_at_start: bool = False):
        if cache_type != "paged":
            raise ValueError("only the paged cache exists here (cache_type='paged')")
        if attn_backend not in ("default", "paged-attn"):
            raise ValueError("one attention backend exists here: 'default' (= 'paged-attn')")
        dev = "cuda:0" if device in ("cuda", "auto", "hip") else device
        require_gpu(dev)
        if random_weights or skip_load:
            from .weights import fill_random_
            from .csrc import lib
            lib.load()
            model = build_model(model_path, dtype, dev)
            tie = bool(getattr(model.config, "tie_word_embeddings", False))
            fill_random_(model, seed, std=random_std, tie=tie)
        else:
            model = load_model(model_path, dtype, dev)
        self.model = model
        self.default_sampling = SamplingParams(temperature=temperature, top_p=top_p, top_k=top_k, max_tokens=max_tokens)
        runner = make_runner(model, num_pages=num_blocks, page_size=block_size, max_requests=max_batch_size,
                             enable_graph=enable_graph, prefix_caching=enable_prefix_caching)
        if max_num_batched_tokens is None:
            env = os.environ.get("INFINILM_MAX_NUM_BATCHED_TOKENS")  # python/infinilm/llm/llm.py:99-102
            max_num_batched_tokens = int(env) if env else model.spec.max_positions
        if tokenizer is None and isinstance(model_path, str):
            tokenizer = _load_tokenizer(model_path)
        self.tokenizer = tokenizer
        self.enable_graph = enable_graph
        if enable_graph and record_graphs_at_start:
            reach = model.spec.max_positions
            if runner.cache.groups:
                # no request holds more than the pool of the group that keeps all keys has (a group that keeps a
                # window needs few pages however long the context: it does not bound the block table's width)
                full = [g for g in runner.cache.groups if g.window <= 0] or runner.cache.groups
                reach = min(reach, max(g.pool.num_pages for g in full) * block_size)
            before = torch.cuda.memory_allocated()
            self.graphs_recorded_at_start = runner.record_decode_graphs(max_batch_size, reach)
            if chunk_size is not None and max_num_batched_tokens < model.spec.max_positions:
                # prompts cut into portions under a token budget: the steps of a busy engine hold the budget's tokens
                self.graphs_recorded_at_start += runner.record_mixed_graphs(max_num_batched_tokens, reach)
            self.graph_memory_bytes = torch.cuda.memory_allocated() - before
            if self.graph_memory_bytes > (4 << 30):
                import warnings
                warnings.warn(f"the {self.graphs_recorded_at_start} decode recordings made at the start hold "
                              f"{self.graph_memory_bytes / 2 ** 30:.1f} GiB of device memory (activations and logits of "
                              "every size); lower max_batch_size or leave record_graphs_at_start off to record sizes as they come",
                              RuntimeWarning)
        self.engine = LLMEngine(runner, max_num_seqs=max_batch_size, max_num_batched_tokens=max_num_batched_tokens,
                                chunk_size=chunk_size, policy=admission, seed=seed, tokenizer=tokenizer,
                                look_ahead=look_ahead)

    def _encode(self, prompt: str) -> List[int]:
        if self.tokenizer is None:
            raise ValueError("this model folder has no tokenizer; pass prompt_token_ids")
        return self.tokenizer.encode(prompt, add_special_tokens=False)

    def generate(self, prompts: Union[str, Sequence[str], None] = None, messages=None,
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 use_tqdm: bool = False, prompt_token_ids: Optional[Sequence[Sequence[int]]] = None) -> List[RequestOutput]:
        if messages is not None:
            return self.chat(messages, sampling_params, use_tqdm)
        if prompt_token_ids is None:
            if prompts is None:
                raise ValueError("give prompts or prompt_token_ids")
            if isinstance(prompts, str):
                prompts = [prompts]
            prompt_token_ids = [self._encode(p) for p in prompts]
            texts = list(prompts)
        else:
            if prompt_token_ids and isinstance(prompt_token_ids[0], int):
                prompt_token_ids = [prompt_token_ids]
            texts = [None] * len(prompt_token_ids)
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            sps = [(sampling_params or self.default_sampling).clone() for _ in prompt_token_ids]
        else:
            sps = list(sampling_params)
            if len(sps) != len(prompt_token_ids):
                raise ValueError("one SamplingParams per prompt, or one for all")
        reqs = [self.engine.add_request(ids, sp, prompt=t) for ids, sp, t in zip(prompt_token_ids, sps, texts)]
        bar = None
        if use_tqdm:
            from tqdm import tqdm
            bar = tqdm(total=len(reqs), desc="requests")
        while any(not r.is_finished() for r in reqs):
            done = self.engine.step()
            if bar is not None:
                bar.update(sum(1 for r in done if r in reqs))
        if bar is not None:
            bar.close()
        return [r.to_request_output() for r in reqs]

    def chat(self, messages, sampling_params=None, use_tqdm: bool = False) -> List[RequestOutput]:
        if self.tokenizer is None:
            raise ValueError("chat needs a tokenizer with a chat template")
        if messages and isinstance(messages[0], dict):
            messages = [messages]
        prompts = [self.tokenizer.apply_chat_template(m, tokenize=False, add_generation_prompt=True) for m in messages]
        return self.generate(prompts, sampling_params=sampling_params, use_tqdm=use_tqdm)

    def close(self) -> None:
        self.engine = None
        self.model = None
        torch.cuda.empty_cache()
