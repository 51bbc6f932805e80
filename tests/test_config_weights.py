"""Configuration, registry, weight loading errors and the random-weights writer (no GPU)."""
import json
import math
import os

import pytest
import torch

import plain_minicpm4 as P
from infinilm_amd.config import ConfigError, load_model_config, registered_architectures
from infinilm_amd.engine.loading import build_model, resolve_dtype
from infinilm_amd.weights import WeightError, load_state_dict, load_weights, random_state_dict, write_random_model


def test_typed_config_reads_the_architectures_own_keys():
    arch, cfg = load_model_config(P.tiny_config_b())
    assert arch.name == "MiniCPMForCausalLM"
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads) == (96, 3, 3, 1)
    assert cfg.head_dim == 32 and cfg.rotary_dim == 32 and cfg.intermediate_size == 200 and cfg.vocab_size == 384
    assert cfg.rope_theta == 50000.0 and cfg.rms_norm_eps == 1e-5 and cfg.max_position_embeddings == 256
    assert cfg.rope_scaling.kind == "longrope" and cfg.rope_scaling.original_max_position_embeddings == 64
    assert len(cfg.rope_scaling.long_factor) == 16 and cfg.rope_scaling.factor == 1.0
    assert cfg.scale_emb == 4 and cfg.residual_scale == pytest.approx(1.0 / math.sqrt(3)) and cfg.logit_scale == 0.5
    assert not cfg.attention_bias and not cfg.mlp_bias and not cfg.attention_output_bias
    # defaults (minicpm4_for_causal_lm.cpp:143-163): head_dim, rope_theta, no scaling, scales of 1
    raw = {k: v for k, v in P.tiny_config_a().items() if k not in ("rope_theta", "scale_emb", "scale_depth", "dim_model_base")}
    _, c2 = load_model_config(raw)
    assert c2.head_dim == 16 and c2.rope_theta == 10000.0 and c2.rope_scaling is None
    assert c2.scale_emb == 1.0 and c2.scale_depth == 1.0 and c2.dim_model_base is None and c2.logit_scale == 1.0
    # `bias` sets both bias keys (:150-153)
    _, c3 = load_model_config(dict(P.tiny_config_a(), bias=True))
    assert c3.attention_bias and c3.mlp_bias and not c3.attention_output_bias


def test_registry_names_and_unknown_architecture():
    assert {"MiniCPMForCausalLM", "minicpm", "minicpm4"} <= set(registered_architectures())
    for raw in ({"model_type": "minicpm4"}, {"model_type": "minicpm"}, {"architectures": ["MiniCPMForCausalLM"], "model_type": "x"}):
        arch, _ = load_model_config(dict(P.tiny_config_a(), **raw))
        assert arch.name == "MiniCPMForCausalLM"
    with pytest.raises(ConfigError, match="Unsupported model_type"):
        load_model_config(dict(P.tiny_config_a(), architectures=["NopeForCausalLM"], model_type="nope"))


@pytest.mark.parametrize("change, match", [
    ({"hidden_size": None}, "Key 'hidden_size' not found"),
    ({"rms_norm_eps": None}, "Key 'rms_norm_eps' not found"),
    ({"max_position_embeddings": None}, "Key 'max_position_embeddings' not found"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"vocab_size": 0}, "must be positive"),
    ({"num_hidden_layers": 2.5}, "must be an integer"),
    ({"hidden_size": "64"}, "must be an integer"),
    ({"rope_scaling": {"type": "bogus"}}, "Unsupported rope_scaling_type"),
    ({"rope_scaling": {"factor": 2}}, "'type' or 'rope_type'"),
    ({"rope_scaling": {"type": "longrope", "short_factor": [1.0] * 8}}, "LongRopeConfig requires"),
    ({"rope_scaling": {"type": "longrope", "short_factor": [1.0] * 7, "long_factor": [1.0] * 8,
                       "original_max_position_embeddings": 64}}, "rotary_dim/2 = 8"),
    ({"rope_scaling": 3}, "must be an object"),
    ({"torch_dtype": "int8"}, "Unsupported dtype"),
    ({"quantization_config": {"bits": 4}}, "quantized"),
    ({"bias": "yes"}, "true or false"),
])
def test_config_errors(change, match):
    raw = P.tiny_config_a()
    for k, v in change.items():
        if v is None:
            raw.pop(k)
        else:
            raw[k] = v
    with pytest.raises(ConfigError, match=match):
        load_model_config(raw)


def test_spec_is_data_and_holds_every_constant():
    arch, cfg = load_model_config(P.tiny_config_b())
    spec = arch.build_spec(cfg)
    assert [r.layer for r in spec.order] == [0, 1, 2] and [r.cache for r in spec.order] == [0, 1, 2]
    m = spec.layers[1].parts["mixer"]
    assert m.kind == "gqa_attention" and m.params["num_heads"] == 3 and m.params["num_kv_heads"] == 1
    assert m.params["scale"] == pytest.approx(1 / math.sqrt(32)) and m.params["window"] == 0
    assert m.params["position"].kind == "rotary" and m.params["position"].params["theta"] == 50000.0
    assert spec.layers[1].parts["ffn"].params == {"hidden_size": 96, "intermediate_size": 200, "bias": False}
    assert spec.layers[0].parts["norm1"].params == {"size": 96, "eps": 1e-5}
    assert spec.embed_scale == 4 and spec.head.scale == 0.5 and spec.layers[0].residual_scale == pytest.approx(3 ** -0.5)


def test_order_validation():
    from infinilm_amd.config import LayerRun
    arch, cfg = load_model_config(P.tiny_config_a())
    spec = arch.build_spec(cfg)
    spec.order = [LayerRun(0, 0), LayerRun(1, 1), LayerRun(0, 2), LayerRun(1, 1, writes_cache=False)]
    spec.validate()  # a layer twice, and a layer reading another run's cache: both are data
    m = build_model(P.tiny_config_a(), "float32", "meta")
    assert len(m.cache_needs) == 2
    spec.order = [LayerRun(0, 0, writes_cache=False)]
    with pytest.raises(ValueError, match="before any run has written"):
        spec.validate()
    spec.order = [LayerRun(0, 0), LayerRun(1, 0)]
    with pytest.raises(ValueError, match="written by"):
        spec.validate()
    spec.order = [LayerRun(5, 0)]
    with pytest.raises(ValueError, match="names layer 5"):
        spec.validate()


def test_dtype_resolution():
    assert resolve_dtype(None, "bfloat16") is torch.bfloat16
    assert resolve_dtype("float32", "bfloat16") is torch.float32
    assert resolve_dtype(None, "float16") is torch.bfloat16
    with pytest.raises(ValueError, match="No dtype"):
        resolve_dtype(None, None)
    with pytest.raises(ValueError, match="Unsupported dtype"):
        resolve_dtype("int4", None)


def _cpu_model(cfg, dtype="float32"):
    return build_model(cfg, dtype, "cpu")


def test_weights_by_name_fused_slices_and_tying():
    cfg = P.tiny_config_a()
    W = P.plain_random_weights(cfg, 1)
    m = _cpu_model(cfg)
    load_state_dict(m, W)
    att = m.blocks[1].mixer
    assert torch.equal(att.qkv.weight[:64], W["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(att.qkv.weight[64:96], W["model.layers.1.self_attn.k_proj.weight"])
    assert torch.equal(att.qkv.weight[96:], W["model.layers.1.self_attn.v_proj.weight"])
    ffn = m.blocks[0].ffn
    assert torch.equal(ffn.gate_up.weight[:128], W["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(ffn.gate_up.weight[128:], W["model.layers.0.mlp.up_proj.weight"])
    assert m.head_is_tied and m.head.data_ptr() == m.embed.data_ptr()
    assert torch.equal(m.embed, W["model.embed_tokens.weight"])  # the scale is not baked into the table
    # untied
    cfgb = P.tiny_config_b()
    Wb = P.plain_random_weights(cfgb, 2)
    mb = _cpu_model(cfgb)
    load_state_dict(mb, Wb)
    assert not mb.head_is_tied and torch.equal(mb.head, Wb["lm_head.weight"])


def test_weight_dtypes_kept():
    cfg = P.tiny_config_a()
    W = P.plain_random_weights(cfg, 1)
    mixed = {k: (v if v.dim() == 1 else v.to(torch.bfloat16)) for k, v in W.items()}
    m = _cpu_model(cfg, "bfloat16")
    load_state_dict(m, mixed)
    assert m.blocks[0].mixer.qkv.weight.dtype == torch.bfloat16 and m.embed.dtype == torch.bfloat16
    assert m.blocks[0].norm1.weight.dtype == torch.float32      # stored in 32-bit: stays so
    assert torch.equal(m.blocks[0].norm1.weight, W["model.layers.0.input_layernorm.weight"])
    m2 = _cpu_model(cfg, "bfloat16")
    load_state_dict(m2, {k: v.to(torch.bfloat16) for k, v in W.items()})
    assert m2.final_norm.weight.dtype == torch.bfloat16          # stored in bfloat16: kept in bfloat16
    m3 = _cpu_model(cfg, "float32")
    load_state_dict(m3, {k: v.to(torch.bfloat16) for k, v in W.items()})
    assert all(p.tensor.dtype == torch.float32 for p in m3.named_parameters().values())


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    cfg = P.tiny_config_b()
    W = P.plain_random_weights(cfg, 3)
    del W["model.layers.2.mlp.up_proj.weight"]
    del W["model.norm.weight"]
    W["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    W["extra.bias"] = torch.zeros(3)
    W["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 96)
    W["lm_head.weight"] = torch.zeros(384, 95)
    with pytest.raises(WeightError) as ei:
        load_state_dict(_cpu_model(cfg), W)
    e = ei.value
    assert sorted(e.missing) == ["model.layers.2.mlp.up_proj.weight", "model.norm.weight"]
    assert sorted(e.unexpected) == ["extra.bias", "model.layers.7.mlp.up_proj.weight"]
    assert len(e.wrong_shape) == 2 and "checkpoint (64, 96), model (32, 96)" in str(e)
    msg = str(e)
    assert "Missing tensor(s) (2)" in msg and "Unexpected tensor(s) (2)" in msg and "Wrong shape(s) (2)" in msg
    # an untied model whose checkpoint lacks both head and embedding: both are reported missing
    W2 = P.plain_random_weights(cfg, 3)
    del W2["lm_head.weight"], W2["model.embed_tokens.weight"]
    with pytest.raises(WeightError) as ei:
        load_state_dict(_cpu_model(cfg), W2)
    assert sorted(ei.value.missing) == ["lm_head.weight", "model.embed_tokens.weight"]


def test_bias_tensors_are_expected_when_config_asks(tmp_path):
    cfg = dict(P.tiny_config_a(), bias=True)
    names = set(_cpu_model(cfg).named_parameters())
    assert "model.layers.0.self_attn.q_proj.bias" in names and "model.layers.1.mlp.down_proj.bias" in names
    assert "model.layers.0.self_attn.o_proj.bias" not in names
    with pytest.raises(WeightError, match="q_proj.bias"):
        load_state_dict(_cpu_model(cfg), P.plain_random_weights(P.tiny_config_a(), 1))


def test_random_model_folder_roundtrip(tmp_path):
    cfg = P.tiny_config_b()
    d = write_random_model(cfg, seed=5, out_dir=str(tmp_path / "m"))
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(d, "config.json")))["hidden_size"] == 96
    m = build_model(d, None, "cpu")
    load_weights(m, d)
    sd = random_state_dict(cfg, 5)
    assert set(sd) == set(P.plain_weight_shapes(cfg))
    assert torch.equal(m.blocks[2].ffn.down.weight, sd["model.layers.2.mlp.down_proj.weight"])
    assert abs(float(sd["model.layers.0.mlp.down_proj.weight"].std()) - 0.02) < 2e-3
    assert not torch.equal(random_state_dict(cfg, 6)["model.norm.weight"], sd["model.norm.weight"])
    # tied configuration: no lm_head in the file
    da = write_random_model(P.tiny_config_a(), seed=5, out_dir=str(tmp_path / "a"), dtype="bfloat16")
    ma = build_model(da, None, "cpu")
    assert ma.dtype == torch.bfloat16
    load_weights(ma, da)
    assert ma.head_is_tied
    with pytest.raises(FileNotFoundError, match="Weight file not found"):
        load_weights(ma, str(tmp_path))


def test_float16_is_run_as_bfloat16_with_a_warning():
    """The reference has float16 as a dtype of its own (csrc/utils.hpp:150-167); this engine says
    aloud that it computes such a model in bfloat16."""
    import torch
    from infinilm_amd.engine.loading import resolve_dtype

    with pytest.warns(RuntimeWarning, match="bfloat16 instead"):
        assert resolve_dtype(None, "float16") == torch.bfloat16
    with pytest.warns(RuntimeWarning, match="bfloat16 instead"):
        assert resolve_dtype("float16", "float32") == torch.bfloat16
    assert resolve_dtype(None, "float32") == torch.float32
    with pytest.raises(ValueError, match="Unsupported dtype"):
        resolve_dtype("int8", None)


def test_llama3_and_yarn_rope_scalings_are_accepted_with_their_keys():
    """The other two kinds the reference's factory knows (rope_scaling_creators.cpp:54-102): keys,
    defaults and error messages as there; the arithmetic is not in the reference's text (parity
    unpinned), so it is pinned here by what the definitions imply: frequencies that turn often stay,
    those that turn seldom are divided by the factor, in between they change monotonically."""
    from infinilm_amd.parts.rotary import SCALINGS

    base = P.tiny_config_a()
    for rs, msg in [({"type": "llama3", "factor": 8.0}, "Llama3RopeScalingConfig requires"),
                    ({"rope_type": "yarn", "factor": 4.0}, "YarnRopeScalingConfig requires")]:
        with pytest.raises(ConfigError, match=msg):
            load_model_config(dict(base, rope_scaling=rs))
    _, cfg = load_model_config(dict(base, rope_scaling={"type": "yarn", "factor": 4.0, "original_max_position_embeddings": 32}))
    assert cfg.rope_scaling.kind == "yarn" and cfg.rope_scaling.extra == {"beta_fast": 32, "beta_slow": 1, "mscale": 1.0,
                                                                          "mscale_all_dim": 0.0}
    m = build_model(dict(base, rope_scaling={"type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                             "original_max_position_embeddings": 64}), "float32", "meta")
    assert m.blocks[0].mixer.position.scaling["high_freq_factor"] == 4.0

    half, theta, orig = 64, 10000.0, 8192
    inv = 1.0 / theta ** (2.0 * torch.arange(half, dtype=torch.float64) / (2 * half))
    new, mag = SCALINGS["llama3"](inv, {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                        "original_max_position_embeddings": orig}, 131072)
    wavelen = 2 * math.pi / inv
    assert mag == 1.0
    assert torch.equal(new[wavelen < orig / 4.0], inv[wavelen < orig / 4.0])
    assert torch.allclose(new[wavelen > orig], inv[wavelen > orig] / 8.0, rtol=1e-12)
    ratio = new / inv
    assert (ratio[1:] <= ratio[:-1] + 1e-12).all() and ratio.min() >= 1 / 8.0 - 1e-12 and ratio.max() <= 1.0

    new, mag = SCALINGS["yarn"](inv, {"factor": 4.0, "original_max_position_embeddings": 4096}, 16384, theta)
    ratio = new / inv
    assert ratio[0] == 1.0 and abs(float(ratio[-1]) - 0.25) < 1e-12 and (ratio[1:] <= ratio[:-1] + 1e-12).all()
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    same, one = SCALINGS["yarn"](inv, {"factor": 1.0, "original_max_position_embeddings": 4096}, 4096, theta)
    assert torch.allclose(same, inv, rtol=1e-12) and one == 1.0
    _, both = SCALINGS["yarn"](inv, {"factor": 4.0, "original_max_position_embeddings": 4096, "mscale": 0.7,
                                     "mscale_all_dim": 0.7}, 16384, theta)
    assert both == 1.0
