"""Plain, slow MiniCPM4 (MiniCPMForCausalLM): whole sequences, no cache, one function per part.

Written from the reference's formulas; every function cites where the reference states what it
computes.  It shares no code with the `infinilm_amd` package: it reads `config.json` keys from a
plain dict and weights from a plain dict of CPU tensors, and computes in float64 by default so that
it can serve as the oracle for both the 32-bit and the bfloat16 engine paths.

Where the reference delegates the arithmetic to its external tensor library (RMSNorm, the rotation,
LongRoPE's factors, SwiGLU, sampling), the definition used here is stated in the docstring and is
pinned by `tests/test_plain.py` through special cases and invariants.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

DT = torch.float64


# --------------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------------
def plain_linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None,
                 alpha: float = 1.0) -> torch.Tensor:
    """y = alpha * (x W^T + b); W is [out, in].

    Layout [out, in]: csrc/layers/quantization/none_quantization.cpp:11-24; call
    `op::linear(x, W, bias, alpha)`: none_quantization.cpp:26-46; alpha member:
    csrc/layers/linear/base_linear.hpp:34-35,69.  How alpha meets a bias is not in the
    reference's text; here the whole branch is scaled.
    """
    y = x @ w.transpose(-1, -2)
    if b is not None:
        y = y + b
    return y * alpha


def plain_embedding(ids: torch.Tensor, table: torch.Tensor, scale_emb: float) -> torch.Tensor:
    """h0 = scale_emb * E[ids].

    Lookup: csrc/models/minicpm4/minicpm4_for_causal_lm.cpp:92; the factor is multiplied into the
    table when weights are loaded: python/infinilm/modeling_utils.py:258-263.
    """
    return table[ids.long()] * scale_emb


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w over the last axis (weight multiplies, no `1 + w`).

    Constructed as RMSNorm(hidden_size, rms_norm_eps): minicpm4_for_causal_lm.cpp:41-45,79,86.
    The formula itself lives in the reference's tensor library; it is pinned in the tests by
    torch.nn.functional.rms_norm and by scale invariance.
    """
    var = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * w


def plain_rotary_dim(cfg: dict) -> int:
    """csrc/config/model_config.cpp:41-57."""
    d = plain_head_dim(cfg)
    f = float(cfg.get("partial_rotary_factor", 1.0))
    if f <= 0.0 or f >= 1.0:
        return d
    rd = int(round(d * f))
    rd = min(max(rd, 2), d)
    if rd % 2:
        rd -= 1
    return max(rd, 2)


def plain_head_dim(cfg: dict) -> int:
    """head_dim defaults to hidden_size / num_attention_heads: minicpm4_for_causal_lm.cpp:143-146."""
    return int(cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]))


def plain_rope_tables(cfg: dict):
    """cos, sin tables [max_position_embeddings, rotary_dim/2] in float64.

    Keys read and their defaults: rope_theta 10000.0 (minicpm4_for_causal_lm.cpp:147-149),
    rope_scaling null/absent = none, type from `type` or `rope_type`
    (csrc/layers/rotary_embedding/rotary_embedding_factory.cpp:11-39); `longrope` needs
    short_factor, long_factor, original_max_position_embeddings, optional factor = 1.0
    (csrc/layers/rotary_embedding/rope_scaling_creators.cpp:23-47).  The table is built once
    for max_position_embeddings positions (rotary_embedding.cpp:90-113), so nothing in it can
    depend on a request's length.

    Definition (the arithmetic is not in the reference's text):
      inv_freq_i = 1 / (f_i * theta^(2i/rd)), i in [0, rd/2)
      f = long_factor if max_position_embeddings > original_max_position_embeddings else short_factor
      s = factor if given and != 1 else max_position_embeddings / original_max_position_embeddings
      m = sqrt(1 + ln(s)/ln(original_max_position_embeddings)) if s > 1 else 1
      cos = m*cos(p*inv_freq), sin = m*sin(p*inv_freq)
    """
    rd = plain_rotary_dim(cfg)
    theta = float(cfg.get("rope_theta", 10000.0))
    max_pos = int(cfg["max_position_embeddings"])
    i = torch.arange(rd // 2, dtype=DT)
    inv_freq = 1.0 / (theta ** (2.0 * i / rd))
    m = 1.0
    rs = cfg.get("rope_scaling")
    if rs is not None:
        kind = rs.get("type", rs.get("rope_type"))
        if kind is None:
            raise ValueError("rope_scaling must contain 'type' or 'rope_type'")
        if kind in ("default", "none", "dynamic"):
            pass
        elif kind == "longrope":
            orig = int(rs["original_max_position_embeddings"])
            factors = rs["long_factor"] if max_pos > orig else rs["short_factor"]
            f = torch.tensor(factors, dtype=DT)
            assert f.numel() == rd // 2
            inv_freq = inv_freq / f
            s = float(rs.get("factor", 1.0))
            if s == 1.0:
                s = max_pos / orig
            if s > 1.0:
                m = math.sqrt(1.0 + math.log(s) / math.log(orig))
        elif kind == "llama3":
            inv_freq = torch.tensor(plain_llama3_frequencies(inv_freq.tolist(), rs), dtype=DT)
        elif kind == "yarn":
            freqs, m = plain_yarn_frequencies(inv_freq.tolist(), rs, rd, theta)
            inv_freq = torch.tensor(freqs, dtype=DT)
        else:
            raise ValueError("Unsupported rope_scaling_type: " + str(kind))
    p = torch.arange(max_pos, dtype=DT)
    ang = p[:, None] * inv_freq[None, :]
    return torch.cos(ang) * m, torch.sin(ang) * m


def plain_llama3_frequencies(inv_freq: Sequence[float], rs: dict) -> list:
    """`llama3` scaling, pair by pair.  Keys (all required): factor, low_freq_factor, high_freq_factor,
    original_max_position_embeddings: rope_scaling_creators.cpp:54-75.  The arithmetic is not in the
    reference's text (it lies in its tensor library): parity unpinned.  Definition used: a pair that
    turns more than high_freq_factor times within the original length keeps its frequency; one that turns
    less than low_freq_factor times has it divided by factor; between the two the division is blended in
    linearly in the number of turns."""
    factor, low, high = float(rs["factor"]), float(rs["low_freq_factor"]), float(rs["high_freq_factor"])
    orig = float(rs["original_max_position_embeddings"])
    out = []
    for w in inv_freq:
        turns = orig * w / (2.0 * math.pi)     # full turns of this pair over the original length
        if turns > high:
            out.append(w)
        elif turns < low:
            out.append(w / factor)
        else:
            t = (turns - low) / (high - low)
            out.append(t * w + (1.0 - t) * w / factor)
    return out


def plain_yarn_frequencies(inv_freq: Sequence[float], rs: dict, rd: int, theta: float):
    """`yarn` scaling, pair by pair; returns (frequencies, magnitude of cos and sin).  Keys and defaults:
    factor and original_max_position_embeddings required, beta_fast 32, beta_slow 1 (cut to whole numbers),
    mscale 1, mscale_all_dim 0, the rotary dim and rope_theta from the model: rope_scaling_creators.cpp:80-102.
    The arithmetic is not in the reference's text: parity unpinned.  Definition used: the pair index at
    which a pair turns beta times within the original length is rd * ln(orig / (2 pi beta)) / (2 ln theta);
    pairs below the index for beta_fast (rounded down, at least 0) keep their frequency, pairs above the
    index for beta_slow (rounded up, at most the last pair) have it divided by factor, a linear ramp
    between; the magnitude is (0.1 mscale ln factor + 1) / (0.1 mscale_all_dim ln factor + 1) for factor > 1."""
    factor, orig = float(rs["factor"]), float(rs["original_max_position_embeddings"])
    beta_fast, beta_slow = int(rs.get("beta_fast", 32)), int(rs.get("beta_slow", 1))

    def index_of(beta):
        return rd * math.log(orig / (2.0 * math.pi * beta)) / (2.0 * math.log(theta))

    first = max(math.floor(index_of(beta_fast)), 0)
    last = min(math.ceil(index_of(beta_slow)), rd // 2 - 1)
    width = max(last - first, 0.001)
    out = []
    for i, w in enumerate(inv_freq):
        stretched = min(max((i - first) / width, 0.0), 1.0)   # 0: kept, 1: divided by factor
        out.append(w * (1.0 - stretched) + (w / factor) * stretched)

    def gain(mscale):
        return 0.1 * mscale * math.log(factor) + 1.0 if factor > 1.0 else 1.0

    return out, gain(float(rs.get("mscale", 1.0))) / gain(float(rs.get("mscale_all_dim", 0.0)))


def plain_apply_rope(x: torch.Tensor, pos: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                     rd: int) -> torch.Tensor:
    """Rotate-half (GPT-NeoX) pairing over the first rd dims of x [T, heads, d].

    Pairing: csrc/config/model_config.hpp:139 (rope_algo GPT_NEOX): dims (i, i + rd/2).
    Applied to q and k after the head view, with per-token positions: attention.cpp:115-129.
      x'[i]        = x[i]*cos_i - x[i+rd/2]*sin_i
      x'[i+rd/2]   = x[i+rd/2]*cos_i + x[i]*sin_i
    """
    c = cos[pos.long()][:, None, :]
    s = sin[pos.long()][:, None, :]
    half = rd // 2
    a = x[..., :half]
    b = x[..., half:rd]
    out = x.clone()
    out[..., :half] = a * c - b * s
    out[..., half:rd] = b * c + a * s
    return out


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                    window: int = 0, first_row: int = 0) -> torch.Tensor:
    """Causal grouped-query attention of one whole sequence.

    q [T, nh, d], k/v [T, nkv, d] -> [T, nh, d].  Query head h uses KV head h // (nh/nkv)
    (contiguous groups), scores = q k^T * scale, causal softmax, P V:
    csrc/layers/attention/backends/static_attn.cpp:82-99; scale = 1/sqrt(head_dim):
    csrc/layers/attention/attention.cpp:41.  `window` > 0 keeps only the last `window` keys
    (this architecture never sets it; the engine's parts take it as a parameter).
    `first_row` > 0 computes (and returns) only the query rows from there on.
    """
    T, nh, d = q.shape
    nkv = k.shape[1]
    g = nh // nkv
    rows = torch.arange(first_row, T, device=q.device)
    out = torch.empty_like(q[first_row:])
    i = torch.arange(T, device=q.device)
    mask = i[None, :] <= rows[:, None]
    if window > 0:
        mask &= i[None, :] > (rows[:, None] - window)
    for h in range(nh):
        kh = h // g
        s = (q[first_row:, h, :] @ k[:, kh, :].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = p @ v[:, kh, :]
    return out


def plain_swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up with silu(x) = x / (1 + exp(-x)).

    csrc/layers/mlp/mlp.cpp:29-38 (`swiglu(up, gate)`, comment "silu(gate) * up"); gate is the
    first half of the fused projection: csrc/layers/linear/fused_linear.cpp:152-158,177-180.
    """
    return gate * torch.sigmoid(gate) * up


def plain_mlp(x, w_gate, w_up, w_down, alpha, b_gate=None, b_up=None, b_down=None):
    """down_proj(silu(gate_proj x) * up_proj x) * alpha: mlp.cpp:29-38; alpha on down_proj:
    minicpm4_for_causal_lm.cpp:30-34."""
    act = plain_swiglu(plain_linear(x, w_gate, b_gate), plain_linear(x, w_up, b_up))
    return plain_linear(act, w_down, b_down, alpha)


def plain_residual_scale(cfg: dict) -> float:
    """scale_depth / sqrt(num_hidden_layers), scale_depth default 1.0:
    minicpm4_for_causal_lm.cpp:12-20."""
    return float(cfg.get("scale_depth", 1.0)) / math.sqrt(float(cfg["num_hidden_layers"]))


def plain_self_attention(x, pos, cfg, W, prefix, cos, sin, alpha, taps=None):
    """qkv projection -> heads -> rotation of q and k -> attention -> o_proj * alpha.

    attention.cpp:96-137; slices in the order q, k, v: fused_linear.cpp:62-71; alpha on o_proj:
    minicpm4_for_causal_lm.cpp:23-28.  Biases exist only when `bias`/`attention_bias`/
    `attention_output_bias` ask for them (minicpm4_for_causal_lm.cpp:150-162).
    """
    nh = int(cfg["num_attention_heads"])
    nkv = int(cfg["num_key_value_heads"])
    d = plain_head_dim(cfg)
    rd = plain_rotary_dim(cfg)
    T = x.shape[0]
    g = lambda n: W.get(prefix + n)
    q = plain_linear(x, W[prefix + "q_proj.weight"], g("q_proj.bias")).view(T, nh, d)
    k = plain_linear(x, W[prefix + "k_proj.weight"], g("k_proj.bias")).view(T, nkv, d)
    v = plain_linear(x, W[prefix + "v_proj.weight"], g("v_proj.bias")).view(T, nkv, d)
    q = plain_apply_rope(q, pos, cos, sin, rd)
    k = plain_apply_rope(k, pos, cos, sin, rd)
    if taps is not None:
        taps[prefix + "q_rotated"] = q.reshape(T, nh * d)
        taps[prefix + "k_rotated"] = k.reshape(T, nkv * d)
        taps[prefix + "v"] = v.reshape(T, nkv * d)
    o = plain_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, nh * d)
    return plain_linear(o, W[prefix + "o_proj.weight"], g("o_proj.bias"), alpha)


# --------------------------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------------------------
def plain_forward(cfg: dict, weights: Dict[str, torch.Tensor], token_ids: Sequence[int],
                  first_position: int = 0, taps: Optional[dict] = None) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence.

    The un-fused form `x = x + f(norm(x))` that the reference states as equal to its fused
    add+norm: minicpm4_for_causal_lm.cpp:59-71 (naive) vs :49-57 (fused); model loop :89-101;
    final norm :99; head with alpha = dim_model_base / hidden_size only when the key exists
    :115-120; a checkpoint without lm_head.weight uses the unscaled embedding table:
    python/infinilm/modeling_utils.py:342-351.
    `first_position` shifts all positions (used to test that only distances count).  `taps`
    receives the residual stream after the embedding ("embed") and after every layer ("layer<l>"),
    and each layer's rotated q, k and its v.  The computation runs where the weights lie.
    """
    W = {k: v.to(DT) for k, v in weights.items()}
    dev = W["model.embed_tokens.weight"].device
    ids = torch.as_tensor(list(token_ids), dtype=torch.long, device=dev)
    T = ids.numel()
    pos = torch.arange(T, device=dev) + first_position
    L = int(cfg["num_hidden_layers"])
    eps = float(cfg["rms_norm_eps"])
    alpha = plain_residual_scale(cfg)
    cos, sin = (t.to(dev) for t in plain_rope_tables(cfg))
    x = plain_embedding(ids, W["model.embed_tokens.weight"], float(cfg.get("scale_emb", 1.0)))
    if taps is not None:
        taps["embed"] = x
    for l in range(L):
        p = f"model.layers.{l}."
        h = plain_rmsnorm(x, W[p + "input_layernorm.weight"], eps)
        x = x + plain_self_attention(h, pos, cfg, W, p + "self_attn.", cos, sin, alpha, taps)
        h = plain_rmsnorm(x, W[p + "post_attention_layernorm.weight"], eps)
        x = x + plain_mlp(h, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"],
                          W[p + "mlp.down_proj.weight"], alpha,
                          W.get(p + "mlp.gate_proj.bias"), W.get(p + "mlp.up_proj.bias"),
                          W.get(p + "mlp.down_proj.bias"))
        if taps is not None:
            taps[f"layer{l}"] = x
    h = plain_rmsnorm(x, W["model.norm.weight"], eps)
    head = W.get("lm_head.weight", W["model.embed_tokens.weight"])
    a_lm = float(cfg["dim_model_base"]) / float(cfg["hidden_size"]) if "dim_model_base" in cfg else 1.0
    return plain_linear(h, head, None, a_lm)


def plain_greedy(cfg: dict, weights, prompt: Sequence[int], n_new: int) -> List[int]:
    """Greedy continuation, recomputing the whole sequence for every token."""
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        logits = plain_forward(cfg, weights, seq)
        t = int(torch.argmax(logits[-1]))
        out.append(t)
        seq.append(t)
    return out


# --------------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------------
def plain_sample_distribution(logits: torch.Tensor, temperature: float, top_k: int,
                              top_p: float) -> torch.Tensor:
    """Probabilities the engine samples from, for one row of logits.

    The reference calls `random_sample_(out, row, random_val, top_p, top_k, temperature)` per
    request (csrc/engine/rank_worker.cpp:467-513); the algorithm is its library's.  Definition
    here: top_k == 1 or temperature == 0 -> all mass on the first argmax; else
    p = softmax(logits / temperature); keep the top_k largest (0 or >= V keeps all; ties with the
    k-th value are kept); then keep the fewest largest whose mass reaches top_p of what is kept
    (ties kept); renormalise.
    """
    l = logits.to(DT)
    V = l.numel()
    if top_k == 1 or temperature == 0.0:
        p = torch.zeros(V, dtype=DT)
        p[int(torch.argmax(l))] = 1.0
        return p
    p = torch.softmax(l / temperature, dim=-1)
    keep = torch.ones(V, dtype=torch.bool)
    if 0 < top_k < V:
        kth = torch.sort(p, descending=True).values[top_k - 1]
        keep &= p >= kth
    if top_p < 1.0:
        pk = torch.where(keep, p, torch.zeros_like(p))
        vals, _ = torch.sort(pk, descending=True)
        csum = torch.cumsum(vals, 0)
        n = int(torch.searchsorted(csum, top_p * pk.sum() * (1 - 1e-12)).item()) + 1
        n = min(n, V)
        keep &= p >= vals[n - 1]
    p = torch.where(keep, p, torch.zeros_like(p))
    return p / p.sum()


def plain_sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float,
                 u: float) -> int:
    """Inverse CDF over the kept tokens in vocabulary order with u in [0, 1)."""
    p = plain_sample_distribution(logits, temperature, top_k, top_p)
    c = torch.cumsum(p, 0)
    idx = int(torch.searchsorted(c, torch.tensor(u, dtype=DT), right=True).item())
    nz = torch.nonzero(p > 0).flatten()
    return min(max(idx, int(nz[0])), int(nz[-1]))


# --------------------------------------------------------------------------------------------
# tiny configurations and random weights for the tests
# --------------------------------------------------------------------------------------------
def tiny_config_a() -> dict:
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "float32",
        "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
        "num_key_value_heads": 2, "intermediate_size": 128, "vocab_size": 256,
        "rope_theta": 10000.0, "max_position_embeddings": 128, "rms_norm_eps": 1e-6,
        "scale_emb": 12, "scale_depth": 1.4, "dim_model_base": 32, "tie_word_embeddings": True,
    }


def tiny_config_b() -> dict:
    g = torch.Generator().manual_seed(77)
    short = (1.0 + torch.rand(16, generator=g)).tolist()
    long = (1.0 + torch.rand(16, generator=g)).tolist()
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "float32",
        "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3,
        "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 200, "vocab_size": 384,
        "rope_theta": 50000.0, "max_position_embeddings": 256, "rms_norm_eps": 1e-5,
        "scale_emb": 4, "scale_depth": 1.0, "dim_model_base": 48, "tie_word_embeddings": False,
        "rope_scaling": {"type": "longrope", "short_factor": short, "long_factor": long,
                         "original_max_position_embeddings": 64},
    }


def tiny_config_c() -> dict:
    """A third shape: nh*d != hidden, head_dim 48 (a multiple of 16, no power of two), no
    dim_model_base, short factors active, odd vocabulary and width."""
    g = torch.Generator().manual_seed(78)
    short = (1.0 + torch.rand(24, generator=g)).tolist()
    long = (2.0 + torch.rand(24, generator=g)).tolist()
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm4", "torch_dtype": "bfloat16",
        "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 6,
        "num_key_value_heads": 3, "head_dim": 48, "intermediate_size": 176, "vocab_size": 331,
        "rope_theta": 20000.0, "max_position_embeddings": 512, "rms_norm_eps": 3e-6,
        "scale_emb": 7, "scale_depth": 2.0, "tie_word_embeddings": True,
        "rope_scaling": {"rope_type": "longrope", "short_factor": short, "long_factor": long,
                         "original_max_position_embeddings": 512},
    }


def tiny_config_d() -> dict:
    """`llama3` scaling whose three bands (kept, blended, divided) all hold pairs of a head of 32; every
    head its own keys."""
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm4", "torch_dtype": "float32",
        "num_hidden_layers": 2, "hidden_size": 72, "num_attention_heads": 3,
        "num_key_value_heads": 3, "head_dim": 32, "intermediate_size": 136, "vocab_size": 211,
        "rope_theta": 10000.0, "max_position_embeddings": 320, "rms_norm_eps": 2e-6,
        "scale_emb": 3, "scale_depth": 1.2, "dim_model_base": 36, "tie_word_embeddings": False,
        "rope_scaling": {"rope_type": "llama3", "factor": 6.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                         "original_max_position_embeddings": 64},
    }


def tiny_config_e() -> dict:
    """`yarn` scaling with a ramp over the middle pairs of a head of 64 and a magnitude other than 1."""
    return {
        "architectures": ["MiniCPMForCausalLM"], "model_type": "minicpm", "torch_dtype": "float32",
        "num_hidden_layers": 2, "hidden_size": 88, "num_attention_heads": 4,
        "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 152, "vocab_size": 173,
        "rope_theta": 5000.0, "max_position_embeddings": 384, "rms_norm_eps": 1e-5,
        "scale_emb": 5, "scale_depth": 1.6, "tie_word_embeddings": True,
        "rope_scaling": {"type": "yarn", "factor": 6.0, "original_max_position_embeddings": 64, "beta_fast": 8,
                         "beta_slow": 1, "mscale": 0.8, "mscale_all_dim": 0.3},
    }


def plain_weight_shapes(cfg: dict) -> Dict[str, tuple]:
    """Tensor names and shapes of a checkpoint of this architecture:
    csrc/models/minicpm4/minicpm4_for_causal_lm.hpp:50-84, attention.cpp:31-37, mlp.cpp:21-26."""
    H = cfg["hidden_size"]
    nh = cfg["num_attention_heads"]
    nkv = cfg["num_key_value_heads"]
    d = plain_head_dim(cfg)
    I = cfg["intermediate_size"]
    V = cfg["vocab_size"]
    s = {"model.embed_tokens.weight": (V, H), "model.norm.weight": (H,)}
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        s[p + "input_layernorm.weight"] = (H,)
        s[p + "post_attention_layernorm.weight"] = (H,)
        s[p + "self_attn.q_proj.weight"] = (nh * d, H)
        s[p + "self_attn.k_proj.weight"] = (nkv * d, H)
        s[p + "self_attn.v_proj.weight"] = (nkv * d, H)
        s[p + "self_attn.o_proj.weight"] = (H, nh * d)
        s[p + "mlp.gate_proj.weight"] = (I, H)
        s[p + "mlp.up_proj.weight"] = (I, H)
        s[p + "mlp.down_proj.weight"] = (H, I)
    if not cfg.get("tie_word_embeddings", False):
        s["lm_head.weight"] = (V, H)
    return s


def plain_random_weights(cfg: dict, seed: int, sharp: bool = True) -> Dict[str, torch.Tensor]:
    """Random float32 weights.  `sharp` makes them so that faults show: norm weights around 1 and
    projections wide enough that attention scores spread over several units, instead of
    N(0, 0.02) everywhere, under which softmax is nearly uniform and rotation errors vanish."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in plain_weight_shapes(cfg).items():
        if len(shape) == 1:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g) if sharp else 0.02 * torch.randn(shape, generator=g)
        else:
            std = (1.5 / math.sqrt(shape[1])) if sharp else 0.02
            if sharp and name.endswith("embed_tokens.weight"):
                std = 1.0 / float(cfg.get("scale_emb", 1.0))
            t = std * torch.randn(shape, generator=g)
        out[name] = t.to(torch.float32)
    return out
