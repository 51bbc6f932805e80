"""Random tiny configurations of the architecture (head counts and groups, head sizes in steps of 16, widths
and vocabularies that are no power of two, biases on either branch, partly rotated heads, LongRoPE or no
scaling, tied or own head, page sizes from 4 to 256) and random ways of cutting a handful of requests into
steps: portions of any size beside decoded tokens, requests left out of steps, up to four live, so few
pages that they are used again.  Every logit against the plain implementation, in 32-bit and in bfloat16.
The committed configurations A, B and C fix three points; this walks between them."""
import json
import os
import random

import pytest
import torch
from safetensors.torch import save_file

import plain_minicpm4 as P
from helpers import TOL, Driver, random_tokens, rel_err

pytestmark = pytest.mark.gpu

def random_config(rng, wide=False):
    """`wide`: widths from 16 and intermediate sizes from 9 on (the committed seeds keep the narrower ranges
    their random streams were drawn with)."""
    nkv = rng.choice([1, 1, 2, 2, 3, 4])
    G = rng.choice([1, 1, 2, 2, 3, 4, 5, 8, 16, 17])
    nh = nkv * G
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    while nh * d > 2048:
        d = rng.choice([16, 32, 48, 64])
    H = 8 * rng.randint(2 if wide else 4, 24)
    I = rng.choice([8 * rng.randint(2 if wide else 4, 40), rng.randint(9 if wide else 33, 300)])
    V = rng.randint(40, 700)
    max_pos = rng.choice([128, 200, 300, 520])
    cfg = {"architectures": ["MiniCPMForCausalLM"], "model_type": rng.choice(["minicpm", "minicpm4"]), "torch_dtype": "float32",
           "num_hidden_layers": rng.randint(1, 3), "hidden_size": H, "num_attention_heads": nh, "num_key_value_heads": nkv,
           "head_dim": d, "intermediate_size": I, "vocab_size": V, "rope_theta": rng.choice([10000.0, 50000.0, 1e6]),
           "max_position_embeddings": max_pos, "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-6]),
           "scale_emb": rng.choice([1, 4, 12]), "scale_depth": rng.choice([1.0, 1.4, 2.0]),
           "tie_word_embeddings": rng.random() < 0.5}
    if rng.random() < 0.6:
        cfg["dim_model_base"] = rng.choice([H // 2, H, 32])
    r = rng.random()
    if r < 0.2:
        cfg["bias"] = True
    elif r < 0.4:
        cfg["attention_bias"] = True
    elif r < 0.5:
        cfg["mlp_bias"] = True
    if rng.random() < 0.25:
        cfg["attention_output_bias"] = True
    if rng.random() < 0.25:
        cfg["partial_rotary_factor"] = 0.5
    rd = int(d * cfg.get("partial_rotary_factor", 1.0))
    r = rng.random()
    g = torch.Generator().manual_seed(rng.randint(0, 1 << 30))
    if r < 0.35:
        cfg["rope_scaling"] = {"type": "longrope", "short_factor": (1.0 + torch.rand(rd // 2, generator=g)).tolist(),
                               "long_factor": (1.5 + torch.rand(rd // 2, generator=g)).tolist(),
                               "original_max_position_embeddings": rng.choice([64, max_pos])}
    return cfg


def weights(cfg, seed):
    """The plain implementation's random weights, and biases where the configuration asks for them."""
    W = P.plain_random_weights(cfg, seed)
    g = torch.Generator().manual_seed(seed + 1)
    nh, nkv, d, H, I = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"], cfg["intermediate_size"]
    att_b = cfg.get("bias", cfg.get("attention_bias", False))
    mlp_b = cfg.get("bias", cfg.get("mlp_bias", False))
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        if att_b:
            for n, s in (("q_proj", nh * d), ("k_proj", nkv * d), ("v_proj", nkv * d)):
                W[p + f"self_attn.{n}.bias"] = 0.3 * torch.randn(s, generator=g)
        if cfg.get("attention_output_bias", False):
            W[p + "self_attn.o_proj.bias"] = 0.3 * torch.randn(H, generator=g)
        if mlp_b:
            W[p + "mlp.gate_proj.bias"] = 0.3 * torch.randn(I, generator=g)
            W[p + "mlp.up_proj.bias"] = 0.3 * torch.randn(I, generator=g)
            W[p + "mlp.down_proj.bias"] = 0.3 * torch.randn(H, generator=g)
    return W


def run_case(seed, tmp, wide=False, tol=TOL):
    """One random configuration, one random schedule; every finished request is compared whole.
    Returns the worst error of the case."""
    rng = random.Random(seed)
    cfg = random_config(rng, wide)
    dtype = rng.choice(["float32", "bfloat16", "bfloat16"])
    page = rng.choice([4, 8, 16, 32, 64, 128, 256])
    print(f"[case] seed {seed} {dtype} page {page} " + json.dumps({k: v for k, v in cfg.items() if k not in ("rope_scaling", "architectures")})
          + " scaling " + str((cfg.get("rope_scaling") or {}).get("type", (cfg.get("rope_scaling") or {}).get("rope_type"))), flush=True)
    W = weights(cfg, seed)
    if dtype == "bfloat16":
        W = {k: v.to(torch.bfloat16) for k, v in W.items()}
    d = str(tmp)
    with open(os.path.join(d, "config.json"), "w") as fh:
        json.dump(dict(cfg, torch_dtype=dtype), fh)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(d, "model.safetensors"), metadata={"format": "pt"})
    Wf = {k: v.to(torch.float32) for k, v in W.items()}
    n_req = rng.randint(3, 7)
    lens = [rng.choice([1, 2, rng.randint(3, 70), rng.randint(60, cfg["max_position_embeddings"])]) for _ in range(n_req)]
    toks = {f"q{i}": random_tokens(cfg, n, seed * 31 + i) for i, n in enumerate(lens)}
    oracle = {r: P.plain_forward(cfg, Wf, t) for r, t in toks.items()}
    need = lambda n: -(-n // page)
    num_pages = sum(sorted((need(n) for n in lens), reverse=True)[:4])
    drv = Driver(d, dtype, num_pages=num_pages, page_size=page)
    waiting = list(toks)
    live = {}
    worst = 0.0
    while waiting or live:
        while waiting and len(live) < 4:
            r = waiting[0]
            held = sum(need(len(toks[x])) for x in live)
            if held + need(len(toks[r])) > num_pages:
                break
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for r in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue   # left out of this step
            left = len(toks[r]) - live[r]
            k = min(left, rng.choice([1, 1, 2, 2, 3, 5, 8, 9, 17, 33, 64, left]))
            entries.append((r, toks[r][live[r]:live[r] + k]))
            live[r] += k
            if live[r] == len(toks[r]):
                end.append(r)
        if not entries:
            continue
        drv.step(entries, end=end)
        for r in end:
            del live[r]
            err = rel_err(drv.request_logits(r, len(toks[r])), oracle[r])
            worst = max(worst, err)
            assert err < tol[dtype], f"seed {seed} ({dtype}, pages of {page}): request {r} of {len(toks[r])} tokens: error {err:.3e}"
    assert drv.runner.cache.free_pages() == num_pages
    print(f"[ok] seed {seed} worst error {worst:.2e}", flush=True)
    return worst


@pytest.mark.parametrize("seed", list(range(48)))
def test_random_configuration_and_random_steps(seed, tmp_path):
    run_case(seed, tmp_path)


# Ten bfloat16 cases that a run of 600 further seeds of the wide generator left beyond the tolerance (4.1e-2 to
# 6.6e-2 against 4e-2): narrow layers (intermediate sizes of 14 to 17 under widths near 100, or a width of 16 to
# 24 under dozens of heads), where one bfloat16 rounding of an activation is a large part of a logit.
ROUNDING_BOUND_SEEDS = [131, 144, 183, 211, 261, 267, 431, 483, 510, 633]


@pytest.mark.parametrize("seed", ROUNDING_BOUND_SEEDS)
def test_cases_beyond_the_tolerance_are_bound_by_rounding_not_by_a_kernel(seed, tmp_path, monkeypatch):
    """The same case through the product kernels and through the plain kernels (the FMA product in ascending
    k, the attention without matrix instructions, no fused epilogue): what exceeds the tolerance must exceed it
    there too, within a factor of 1.5; a fault of a product kernel would stand out against the plain ones."""
    from infinilm_amd import kernels

    loose = {"float32": TOL["float32"], "bfloat16": 1.0}
    product = run_case(seed, tmp_path, wide=True, tol=loose)
    monkeypatch.setattr(kernels, "FORCE_BASIC", True)
    plain = run_case(seed, tmp_path, wide=True, tol=loose)
    print(f"[err] seed {seed}: product kernels {product:.3e}, plain kernels {plain:.3e}", flush=True)
    assert product <= 1.5 * plain, f"seed {seed}: product kernels {product:.3e} against plain kernels {plain:.3e}"
