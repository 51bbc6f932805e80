"""config.json contents of the model shapes the benchmarks run with random weights: the MiniCPM4-8B,
MiniCPM4-0.5B and MiniCPM-2B-family layer sizes.  LongRoPE factors are drawn from a fixed seed
(uniform in [1, 4]); nothing else is random."""
from __future__ import annotations


def _factors(n: int, seed: int):
    import torch
    g = torch.Generator().manual_seed(seed)
    short = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    long = (1.0 + 3.0 * torch.rand(n, generator=g)).tolist()
    return short, long


def shape_config(name: str, layers: int = 0) -> dict:
    """`name`: "8b", "0.5b" or "2b"; `layers` > 0 overrides the number of layers."""
    base = {"architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "bfloat16", "rope_theta": 10000.0,
            "scale_emb": 12, "scale_depth": 1.4, "dim_model_base": 256}
    if name == "8b":
        short, long = _factors(64, 1234)
        cfg = dict(base, num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=2, head_dim=128,
                   intermediate_size=16384, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=False,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "0.5b":
        short, long = _factors(32, 1235)
        cfg = dict(base, num_hidden_layers=24, hidden_size=1024, num_attention_heads=16, num_key_value_heads=2, head_dim=64,
                   intermediate_size=4096, vocab_size=73448, max_position_embeddings=32768, rms_norm_eps=1e-6,
                   tie_word_embeddings=True,
                   rope_scaling={"type": "longrope", "short_factor": short, "long_factor": long,
                                 "original_max_position_embeddings": 32768})
    elif name == "2b":
        cfg = dict(base, num_hidden_layers=40, hidden_size=2304, num_attention_heads=36, num_key_value_heads=36, head_dim=64,
                   intermediate_size=5760, vocab_size=122753, max_position_embeddings=4096, rms_norm_eps=1e-5,
                   tie_word_embeddings=True)
    else:
        raise KeyError(f"unknown shape {name!r}; there are 8b, 0.5b and 2b")
    if layers > 0:
        cfg["num_hidden_layers"] = int(layers)
    return cfg
