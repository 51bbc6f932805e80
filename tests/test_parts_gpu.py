"""Each part of a layer alone against the plain implementation, and the generality of the parts:
a window mixer whose pages are given back, a layer order that names a layer twice and lets a layer
read another layer's cache, and a toy mixer with state of its own that is defined here, registered
from here, built and stepped without a change to the framework's files."""
import json
import math
import os

import pytest
import torch

import plain_minicpm4 as P
from helpers import rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


def _ctx(dtype):
    from infinilm_amd.parts import BuildContext
    return BuildContext(dtype=dtype, device=torch.device(DEV))


def _fill(part, seed, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, p in sorted(part.named_parameters().items()):
        t = torch.randn(tuple(p.tensor.shape), generator=g) * scale
        if t.dim() == 1:
            t = t + 1.0
        t = t.to(p.tensor.dtype)
        p.tensor.copy_(t)
        W[name] = t.to(F64)
    return W


class _Harness:
    """A cache manager and step batches for one mixer, without a model around it."""

    def __init__(self, needs, dtype, page_size=8, num_pages=32):
        from infinilm_amd.cache import CacheManager
        from infinilm_amd.engine.step import StepRunner

        class _Spec:
            vocab_size = 1 << 30
            max_positions = 1 << 20

        class _Model:
            spec = _Spec()
            device = torch.device(DEV)

        self.cache = CacheManager(needs, page_size=page_size, num_pages=num_pages, max_requests=4, dtype=dtype, device=DEV)
        self.runner = StepRunner(_Model(), self.cache)

    def batch(self, entries):
        from infinilm_amd.engine.step import StepEntry
        for rid, n in entries:
            if not self.cache.has(rid):
                self.cache.admit(rid)
        b = self.runner.build_batch([StepEntry(rid, [0] * n, []) for rid, n in entries])
        return b

    def commit(self, entries):
        for rid, n in entries:
            self.cache.commit(rid, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from infinilm_amd.parts import ResidualStream
    from infinilm_amd.parts.registry import build_norm
    from infinilm_amd.config import PartSpec

    norm = build_norm(PartSpec("rmsnorm", {"size": 96, "eps": 1e-5}), _ctx(dtype))
    W = _fill(norm, 1)
    r = torch.randn(6, 96)
    h = torch.randn(6, 96).to(dtype)
    stream = ResidualStream(r.to(DEV).clone())
    stream.push(h.to(DEV), 0.7)
    x = norm.forward(stream)
    assert stream.pending is None
    want_r = r.to(F64) + 0.7 * h.to(F64)
    assert rel_err(stream.residual, want_r) < 1e-6
    assert rel_err(x, P.plain_rmsnorm(want_r, W["weight"], 1e-5)) < (2e-6 if dtype == torch.float32 else 1e-2)


def test_rotary_part_tables():
    from infinilm_amd.parts.registry import build_position_encoding
    from infinilm_amd.config import PartSpec

    for make in (P.tiny_config_a, P.tiny_config_b, P.tiny_config_c):
        cfg = make()
        d = P.plain_head_dim(cfg)
        rope = build_position_encoding(PartSpec("rotary", {"head_dim": d, "rotary_dim": d,
                                                           "max_positions": cfg["max_position_embeddings"],
                                                           "theta": cfg["rope_theta"], "scaling": cfg.get("rope_scaling")}),
                                       _ctx(torch.float32))
        cos, sin = P.plain_rope_tables(cfg)
        assert rope.cos.dtype == torch.float32 and tuple(rope.cos.shape) == tuple(cos.shape)
        assert rel_err(rope.cos, cos) < 1e-6 and rel_err(rope.sin, sin) < 1e-6
    with pytest.raises(ValueError, match="Unsupported rope_scaling_type"):
        build_position_encoding(PartSpec("rotary", {"head_dim": 16, "rotary_dim": 16, "max_positions": 8, "theta": 1e4,
                                                    "scaling": {"type": "bogus"}}), _ctx(torch.float32))


@pytest.mark.parametrize("dtype,page", [(torch.float32, 8), (torch.bfloat16, 16)])
@pytest.mark.parametrize("window", [0, 13])
def test_attention_part_alone_in_portions(dtype, page, window):
    """The mixer alone: a sequence fed in portions through the paged cache equals the plain
    attention over the whole sequence; with a window, pages the window has passed are given back."""
    from infinilm_amd.parts.registry import build_mixer
    from infinilm_amd.config import PartSpec

    H, nh, nkv, d, n = 40, 6, 2, 16, 75
    rope_cfg = {"hidden_size": d, "num_attention_heads": 1, "rope_theta": 999.0, "max_position_embeddings": 128}
    pos = PartSpec("rotary", {"head_dim": d, "rotary_dim": d, "max_positions": 128, "theta": 999.0, "scaling": None})
    att = build_mixer(PartSpec("gqa_attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                 "qkv_bias": True, "out_bias": False, "scale": 0.3, "window": window,
                                                 "position": pos}), _ctx(dtype))
    W = _fill(att, 3)
    hz = _Harness([att.cache_need()], dtype, page_size=page, num_pages=12)
    x = (torch.randn(n, H) * 0.8).to(dtype)
    outs, i = [], 0
    for k in (17, 2, 1, 30, 1, 1, 23):
        b = hz.batch([("r", k)])
        o = att.forward(x[i:i + k].to(DEV), b, hz.cache.view(0, b, True))
        outs.append(o.sum(0).to(dtype) if o.dim() == 3 else o.to(dtype))   # a branch may come in float32 parts
        hz.commit([("r", k)])
        i += k
    got = torch.cat(outs)
    # plain: projections, rotation, windowed causal attention, output projection
    xd = x.to(F64)
    cos, sin = P.plain_rope_tables(rope_cfg)
    q = P.plain_linear(xd, W["q_proj.weight"], W["q_proj.bias"]).view(n, nh, d)
    k_ = P.plain_linear(xd, W["k_proj.weight"], W["k_proj.bias"]).view(n, nkv, d)
    v = P.plain_linear(xd, W["v_proj.weight"], W["v_proj.bias"]).view(n, nkv, d)
    p = torch.arange(n)
    o = P.plain_attention(P.plain_apply_rope(q, p, cos, sin, d), P.plain_apply_rope(k_, p, cos, sin, d), v, 0.3, window)
    want = P.plain_linear(o.reshape(n, nh * d), W["o_proj.weight"])
    assert rel_err(got, want) < (5e-6 if dtype == torch.float32 else 2e-2)
    table = hz.cache.table("r", 0)
    if window:
        first = (n - window + 1) // page
        assert all(t == -1 for t in table[:first]) and all(t >= 0 for t in table[first:])
        assert hz.cache.free_pages() == 12 - (len(table) - first)
    else:
        assert all(t >= 0 for t in table)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from infinilm_amd.parts.registry import build_feed_forward
    from infinilm_amd.config import PartSpec

    ffn = build_feed_forward(PartSpec("swiglu", {"hidden_size": 80, "intermediate_size": 200, "bias": True}), _ctx(dtype))
    W = _fill(ffn, 5)
    for rows in (3, 70):   # the few-rows and the many-rows products
        x = torch.randn(rows, 80).to(dtype)
        got = ffn.forward(x.to(DEV), None)
        want = P.plain_mlp(x.to(F64), W["gate_proj.weight"], W["up_proj.weight"], W["down_proj.weight"], 1.0,
                           W["gate_proj.bias"], W["up_proj.bias"], W["down_proj.bias"])
        assert rel_err(got, want) < (5e-6 if dtype == torch.float32 else 2e-2)


# ------------------------------------------------------------------------------------------------
# a toy architecture, defined and registered here
# ------------------------------------------------------------------------------------------------
def _register_toy():
    from infinilm_amd.cache import FixedState
    from infinilm_amd.config import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinilm_amd.parts import Mixer, Param, register_mixer

    @register_mixer("toy_decay")
    class ToyDecayMixer(Mixer):
        """s_t = decay * s_{t-1} + x_t Wi^T (one state row per request), y_t = s_t Wo^T.
        Plain tensor ops stand in for kernels: it is a toy that shows the interfaces."""

        def __init__(self, hidden_size, state_size, decay, ctx):
            self.decay = float(decay)
            self.state_size = int(state_size)
            self.wi = torch.empty((state_size, hidden_size), dtype=ctx.dtype, device=ctx.device)
            self.wo = torch.empty((hidden_size, state_size), dtype=ctx.dtype, device=ctx.device)

        def named_parameters(self):
            return {"in_proj.weight": Param(self.wi), "out_proj.weight": Param(self.wo)}

        def cache_need(self):
            return FixedState((self.state_size,), torch.float32)

        def forward(self, x, batch, view):
            u = x.float() @ self.wi.float().t()
            if batch.all_decode:
                # one token a request: rows by the device's index tensors, so that the step can be recorded
                # as a graph and replayed for other requests (the host copies below would be baked in)
                s = self.decay * view.pool.index_select(0, view.state_in.long()) + u
                view.pool.index_copy_(0, view.state_out.long(), s)
                return (s @ self.wo.float().t()).to(x.dtype)
            out = torch.empty_like(u)
            off = batch.h_seg_offsets
            for i in range(batch.R):
                s = view.pool[int(batch.h_state_in[i])].clone()
                for t in range(int(off[i]), int(off[i + 1])):
                    s = self.decay * s + u[t]
                    out[t] = s
                view.pool[int(batch.h_state_out[i])] = s
            return (out @ self.wo.float().t()).to(x.dtype)

    def config_from_dict(raw):
        return dict(raw)

    def build_spec(cfg):
        H, d = cfg["hidden_size"], cfg["head_dim"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": cfg["eps"]})
        pos = PartSpec("rotary", {"head_dim": d, "rotary_dim": d, "max_positions": cfg["max_positions"], "theta": 1e4,
                                  "scaling": None})
        att = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": cfg["heads"], "num_kv_heads": cfg["kv_heads"],
                                         "head_dim": d, "qkv_bias": False, "out_bias": False, "scale": d ** -0.5,
                                         "window": 0, "position": pos})
        toy = PartSpec("toy_decay", {"hidden_size": H, "state_size": cfg["state_size"], "decay": cfg["decay"]})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg["intermediate_size"], "bias": False})
        names = {"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "ffn": "ffn"}
        mixers = [att, toy, att]
        layers = [LayerSpec(f"blocks.{i}", "pre_norm", {"norm1": norm, "mixer": m, "norm2": norm, "ffn": ffn}, names, 0.5)
                  for i, m in enumerate(mixers)]
        # layer 1 (the toy mixer) runs twice with states of its own; layer 2 reads layer 0's keys and values
        order = [LayerRun(0, 0), LayerRun(1, 1), LayerRun(2, 0, writes_cache=False), LayerRun(1, 2)]
        return ModelSpec("ToyForCausalLM", cfg["vocab_size"], H, cfg["max_positions"], "emb", 1.0, layers, order, norm,
                         "ln_f", HeadSpec("head", 1.0, True))

    register_architecture(["ToyForCausalLM"], config_from_dict, build_spec)


def _toy_plain(cfg, W, ids):
    """The toy model, whole sequence, in float64."""
    W = {k: v.to(F64) for k, v in W.items()}
    n, H, d, nh, nkv = len(ids), cfg["hidden_size"], cfg["head_dim"], cfg["heads"], cfg["kv_heads"]
    cos, sin = P.plain_rope_tables({"hidden_size": d, "num_attention_heads": 1, "max_position_embeddings": cfg["max_positions"]})
    pos = torch.arange(n)
    x = W["emb.weight"][torch.tensor(ids)]
    kv0 = None

    def toy(h, p):
        u = h @ W[p + "in_proj.weight"].T
        s = torch.zeros(cfg["state_size"], dtype=F64)
        out = []
        for t in range(n):
            s = cfg["decay"] * s + u[t]
            out.append(s)
        return torch.stack(out) @ W[p + "out_proj.weight"].T

    for layer, reads_layer0 in ((0, False), (1, None), (2, True), (1, None)):
        p = f"blocks.{layer}."
        h = P.plain_rmsnorm(x, W[p + "ln1.weight"], cfg["eps"])
        if reads_layer0 is None:
            y = toy(h, p + "mix.")
        else:
            q = P.plain_apply_rope(P.plain_linear(h, W[p + "mix.q_proj.weight"]).view(n, nh, d), pos, cos, sin, d)
            if not reads_layer0:
                k = P.plain_apply_rope(P.plain_linear(h, W[p + "mix.k_proj.weight"]).view(n, nkv, d), pos, cos, sin, d)
                v = P.plain_linear(h, W[p + "mix.v_proj.weight"]).view(n, nkv, d)
                kv0 = (k, v)
            o = P.plain_attention(q, kv0[0], kv0[1], d ** -0.5).reshape(n, nh * d)
            y = P.plain_linear(o, W[p + "mix.o_proj.weight"])
        x = x + 0.5 * y
        h = P.plain_rmsnorm(x, W[p + "ln2.weight"], cfg["eps"])
        x = x + 0.5 * P.plain_mlp(h, W[p + "ffn.gate_proj.weight"], W[p + "ffn.up_proj.weight"], W[p + "ffn.down_proj.weight"], 1.0)
    return P.plain_linear(P.plain_rmsnorm(x, W["ln_f.weight"], cfg["eps"]), W["emb.weight"])


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    from safetensors.torch import save_file
    from infinilm_amd.engine.loading import build_model
    from helpers import Driver

    _register_toy()
    cfg = {"architectures": ["ToyForCausalLM"], "torch_dtype": "float32", "vocab_size": 97, "hidden_size": 48,
           "head_dim": 16, "heads": 4, "kv_heads": 2, "intermediate_size": 72, "state_size": 24, "decay": 0.9,
           "eps": 1e-5, "max_positions": 256}
    d = str(tmp_path / "toy")
    os.makedirs(d)
    json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
    meta = build_model(cfg, "float32", "meta")
    names = meta.named_parameters()
    assert "blocks.1.mix.in_proj.weight" in names and "blocks.2.mix.q_proj.weight" in names
    g = torch.Generator().manual_seed(4)
    W = {}
    for name, p in sorted(names.items()):
        if name == "head.weight":
            continue   # tied to the embedding
        t = torch.randn(tuple(p.tensor.shape), generator=g) * (0.3 if len(p.tensor.shape) == 2 else 0.1)
        W[name] = (t + 1.0) if t.dim() == 1 else t
    save_file(W, os.path.join(d, "model.safetensors"), metadata={"format": "pt"})

    drv = Driver(d, "float32", num_pages=24, page_size=8, max_requests=3)
    from infinilm_amd.cache import FixedState, PagedKV
    needs = drv.model.cache_needs
    assert isinstance(needs[0], PagedKV) and isinstance(needs[1], FixedState) and isinstance(needs[2], FixedState)
    g2 = torch.Generator().manual_seed(9)
    seqs = {r: torch.randint(0, 97, (n,), generator=g2).tolist() for r, n in (("a", 50), ("b", 21), ("c", 33))}
    # a in portions, b whole beside a's portions, then c in a slot that b has given back
    drv.step([("a", seqs["a"][:20])])
    drv.step([("a", seqs["a"][20:22]), ("b", seqs["b"])], end=["b"])
    drv.step([("a", seqs["a"][22:23]), ("c", seqs["c"][:5])])
    drv.step([("c", seqs["c"][5:]), ("a", seqs["a"][23:])], end=["a", "c"])
    for r, ids in seqs.items():
        err = rel_err(drv.request_logits(r, len(ids)), _toy_plain(cfg, W, ids))
        assert err < 1e-4, f"request {r}: error {err:.3e}"
    assert drv.runner.cache.free_pages() == 24


def test_attention_without_rotation_is_the_library_routine():
    """Position encoding `none`: the mixer reduces to projections around plain causal attention."""
    import torch.nn.functional as F
    from infinilm_amd.parts.registry import build_mixer
    from infinilm_amd.config import PartSpec

    H, nh, nkv, d, n = 48, 4, 4, 16, 40
    att = build_mixer(PartSpec("gqa_attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                 "qkv_bias": False, "out_bias": False, "scale": d ** -0.5, "window": 0,
                                                 "position": PartSpec("none", {"head_dim": d})}), _ctx(torch.float32))
    W = _fill(att, 11)
    hz = _Harness([att.cache_need()], torch.float32, page_size=8, num_pages=8)
    x = torch.randn(n, H)
    b = hz.batch([("r", n)])
    got = att.forward(x.to(DEV), b, hz.cache.view(0, b, True))
    xd = x.to(F64)
    q, k, v = (F.linear(xd, W[f"{p}_proj.weight"]).view(n, nh, d).transpose(0, 1) for p in "qkv")
    o = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(0, 1).reshape(n, nh * d)
    assert rel_err(got, F.linear(o, W["o_proj.weight"])) < 5e-6


def test_a_rope_scaling_registered_from_outside():
    """Another scaling of the rotary encoding is one registered function; the mixer needs no change."""
    from infinilm_amd.parts import register_rope_scaling
    from infinilm_amd.parts.registry import build_position_encoding
    from infinilm_amd.config import PartSpec

    @register_rope_scaling("toy_linear")
    def _linear(inv_freq, params, max_positions):
        return inv_freq / float(params["factor"]), 1.0

    rope = build_position_encoding(PartSpec("rotary", {"head_dim": 32, "rotary_dim": 16, "max_positions": 64, "theta": 100.0,
                                                       "scaling": {"type": "toy_linear", "factor": 4.0}}), _ctx(torch.float32))
    i = torch.arange(8, dtype=F64)
    ang = torch.arange(64, dtype=F64)[:, None] * (1.0 / (4.0 * 100.0 ** (2 * i / 16)))[None, :]
    assert rel_err(rope.cos, torch.cos(ang)) < 1e-6 and rel_err(rope.sin, torch.sin(ang)) < 1e-6


def test_toy_feed_forward_with_routing(tmp_path):
    """A feed-forward that routes every token to one of three experts, defined and registered here,
    in a model whose layers use different feed-forwards; portions and batches give the whole-sequence result."""
    from safetensors.torch import save_file
    from infinilm_amd import kernels
    from infinilm_amd.config import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinilm_amd.engine.loading import build_model
    from infinilm_amd.parts import FeedForward, Param, register_feed_forward
    from helpers import Driver

    @register_feed_forward("toy_top1_experts")
    class ToyExperts(FeedForward):
        def __init__(self, hidden_size, intermediate_size, num_experts, ctx):
            self.E = int(num_experts)
            self.router = torch.empty((self.E, hidden_size), dtype=torch.float32, device=ctx.device)
            self.gate_up = [torch.empty((2 * intermediate_size, hidden_size), dtype=ctx.dtype, device=ctx.device) for _ in range(self.E)]
            self.down = [torch.empty((hidden_size, intermediate_size), dtype=ctx.dtype, device=ctx.device) for _ in range(self.E)]

        def named_parameters(self):
            out = {"router.weight": Param(self.router)}
            for e in range(self.E):
                out[f"experts.{e}.gate_up.weight"] = Param(self.gate_up[e])
                out[f"experts.{e}.down.weight"] = Param(self.down[e])
            return out

        def forward(self, x, batch):
            choice = kernels.argmax(kernels.gemm(x.float(), self.router)).long()   # router logits in float32
            out = torch.zeros_like(x)
            for e in range(self.E):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel():
                    xe = x.index_select(0, rows).contiguous()
                    out.index_copy_(0, rows, kernels.gemm(kernels.swiglu(kernels.gemm(xe, self.gate_up[e])), self.down[e]))
            return out

    def build_spec(cfg):
        H, d = cfg["hidden_size"], cfg["head_dim"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-6})
        pos = PartSpec("rotary", {"head_dim": d, "rotary_dim": d, "max_positions": 128, "theta": 1e4, "scaling": None})
        att = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": d, "qkv_bias": False,
                                         "out_bias": False, "scale": d ** -0.5, "window": 0, "position": pos})
        dense = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 40, "bias": False})
        moe = PartSpec("toy_top1_experts", {"hidden_size": H, "intermediate_size": 24, "num_experts": 3})
        names = {"norm1": "ln1", "mixer": "att", "norm2": "ln2", "ffn": "ffn"}
        layers = [LayerSpec(f"l.{i}", "pre_norm", {"norm1": norm, "mixer": att, "norm2": norm, "ffn": f}, names, 1.0)
                  for i, f in enumerate([dense, moe])]
        return ModelSpec("ToyRoutedLM", cfg["vocab_size"], H, 128, "emb", 1.0, layers, [LayerRun(0, 0), LayerRun(1, 1)], norm,
                         "ln_f", HeadSpec("head", 1.0, True))

    register_architecture(["ToyRoutedLM"], dict, build_spec)
    cfg = {"architectures": ["ToyRoutedLM"], "torch_dtype": "float32", "vocab_size": 61, "hidden_size": 32, "head_dim": 16}
    d = str(tmp_path / "routed")
    os.makedirs(d)
    json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
    g = torch.Generator().manual_seed(8)
    W = {}
    for name, p in sorted(build_model(cfg, "float32", "meta").named_parameters().items()):
        if name == "head.weight":
            continue
        t = torch.randn(tuple(p.tensor.shape), generator=g) * 0.4
        W[name] = (t * 0.25 + 1.0) if t.dim() == 1 else t
    save_file(W, os.path.join(d, "model.safetensors"), metadata={"format": "pt"})

    def plain(ids):
        Wd = {k: v.to(F64) for k, v in W.items()}
        n = len(ids)
        cos, sin = P.plain_rope_tables({"hidden_size": 16, "num_attention_heads": 1, "max_position_embeddings": 128})
        pos = torch.arange(n)
        x = Wd["emb.weight"][torch.tensor(ids)]
        for l in range(2):
            p = f"l.{l}."
            h = P.plain_rmsnorm(x, Wd[p + "ln1.weight"], 1e-6)
            q = P.plain_apply_rope(P.plain_linear(h, Wd[p + "att.q_proj.weight"]).view(n, 2, 16), pos, cos, sin, 16)
            k = P.plain_apply_rope(P.plain_linear(h, Wd[p + "att.k_proj.weight"]).view(n, 1, 16), pos, cos, sin, 16)
            v = P.plain_linear(h, Wd[p + "att.v_proj.weight"]).view(n, 1, 16)
            x = x + P.plain_linear(P.plain_attention(q, k, v, 0.25).reshape(n, 32), Wd[p + "att.o_proj.weight"])
            h = P.plain_rmsnorm(x, Wd[p + "ln2.weight"], 1e-6)
            if l == 0:
                x = x + P.plain_mlp(h, Wd[p + "ffn.gate_proj.weight"], Wd[p + "ffn.up_proj.weight"], Wd[p + "ffn.down_proj.weight"], 1.0)
            else:
                choice = torch.argmax(h @ Wd[p + "ffn.router.weight"].T, dim=-1)
                y = torch.zeros_like(h)
                for t in range(n):
                    gu = Wd[p + f"ffn.experts.{int(choice[t])}.gate_up.weight"]
                    y[t] = P.plain_mlp(h[t:t + 1], gu[:24], gu[24:], Wd[p + f"ffn.experts.{int(choice[t])}.down.weight"], 1.0)[0]
                x = x + y
        return P.plain_linear(P.plain_rmsnorm(x, Wd["ln_f.weight"], 1e-6), Wd["emb.weight"])

    drv = Driver(d, "float32", num_pages=16, page_size=8, max_requests=2)
    g2 = torch.Generator().manual_seed(3)
    a, b = (torch.randint(0, 61, (n,), generator=g2).tolist() for n in (45, 20))
    drv.step([("a", a[:17])])
    drv.step([("a", a[17:19]), ("b", b)], end=["b"])
    drv.step([("a", a[19:])], end=["a"])
    assert rel_err(drv.request_logits("a", 45), plain(a)) < 1e-4
    assert rel_err(drv.request_logits("b", 20), plain(b)) < 1e-4


def test_a_position_encoding_and_an_output_head_registered_from_outside(tmp_path):
    """Another position encoding, defined here with a tensor of its own (a learned vector per
    position added to every q and k head), and another output head (logits capped by a tanh):
    registered, named in the model's description, loaded by name and stepped in portions and
    batches, without a change to the mixer, the model or the step function."""
    from safetensors.torch import save_file
    from infinilm_amd import kernels
    from infinilm_amd.config import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinilm_amd.engine.loading import build_model
    from infinilm_amd.parts import Param, PositionEncoding, register_head, register_position_encoding
    from infinilm_amd.parts.ends import LinearHead
    from helpers import Driver

    @register_head("toy_capped")
    class ToyCappedHead(LinearHead):
        def __init__(self, vocab_size, hidden_size, scale, cap, ctx):
            super().__init__(vocab_size, hidden_size, scale, ctx)
            self.cap = float(cap)

        def forward(self, x):
            return self.cap * torch.tanh(super().forward(x) / self.cap)

    @register_position_encoding("toy_learned_offsets")
    class ToyLearnedOffsets(PositionEncoding):
        def __init__(self, head_dim, max_positions, ctx):
            self.head_dim, self.max_positions = int(head_dim), int(max_positions)
            self.table = torch.empty((self.max_positions, self.head_dim), dtype=ctx.dtype, device=ctx.device)
            self._none = torch.zeros((1, 0), dtype=torch.float32, device=ctx.device)

        def named_parameters(self):
            return {"offsets.weight": Param(self.table)}

        def encode_and_store(self, qkv, batch, view, nh, nkv, d):
            add = self.table[batch.positions.long()]                       # [T, d]
            heads = qkv[:, :(nh + nkv) * d].view(-1, nh + nkv, d)           # q and k heads, not v
            heads += add[:, None, :]
            # the write alone: the rotation kernel over no dims
            kernels.rope_kvwrite(qkv, batch.positions, self._none, self._none, view.k, view.v, view.slots, nh, nkv, d, 0)

    H, d, nh, nkv, V, MAXP = 32, 16, 4, 2, 53, 96

    def build_spec(cfg):
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-6})
        pos = PartSpec("toy_learned_offsets", {"head_dim": d, "max_positions": MAXP})
        att = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "qkv_bias": False,
                                         "out_bias": False, "scale": d ** -0.5, "window": 0, "position": pos})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 40, "bias": False})
        names = {"norm1": "ln1", "mixer": "att", "norm2": "ln2", "ffn": "ffn"}
        layers = [LayerSpec(f"l.{i}", "pre_norm", {"norm1": norm, "mixer": att, "norm2": norm, "ffn": ffn}, names, 1.0) for i in range(2)]
        return ModelSpec("ToyOffsetsLM", V, H, MAXP, "emb", 1.0, layers, [LayerRun(0, 0), LayerRun(1, 1)], norm, "ln_f",
                         HeadSpec("head", 0.5, True, kind="toy_capped", params={"cap": 3.0}))

    register_architecture(["ToyOffsetsLM"], dict, build_spec)
    cfg = {"architectures": ["ToyOffsetsLM"], "torch_dtype": "float32"}
    mdir = str(tmp_path / "offsets")
    os.makedirs(mdir)
    json.dump(cfg, open(os.path.join(mdir, "config.json"), "w"))
    names = build_model(cfg, "float32", "meta").named_parameters()
    assert "l.1.att.position.offsets.weight" in names
    g = torch.Generator().manual_seed(12)
    W = {}
    for name, p in sorted(names.items()):
        if name == "head.weight":
            continue
        t = torch.randn(tuple(p.tensor.shape), generator=g) * 0.4
        W[name] = (t * 0.25 + 1.0) if t.dim() == 1 else t
    save_file(W, os.path.join(mdir, "model.safetensors"), metadata={"format": "pt"})

    def plain(ids):
        Wd = {k: v.to(F64) for k, v in W.items()}
        n = len(ids)
        x = Wd["emb.weight"][torch.tensor(ids)]
        for l in range(2):
            p = f"l.{l}."
            h = P.plain_rmsnorm(x, Wd[p + "ln1.weight"], 1e-6)
            off = Wd[p + "att.position.offsets.weight"][:n][:, None, :]
            q = P.plain_linear(h, Wd[p + "att.q_proj.weight"]).view(n, nh, d) + off
            k = P.plain_linear(h, Wd[p + "att.k_proj.weight"]).view(n, nkv, d) + off
            v = P.plain_linear(h, Wd[p + "att.v_proj.weight"]).view(n, nkv, d)
            x = x + P.plain_linear(P.plain_attention(q, k, v, d ** -0.5).reshape(n, nh * d), Wd[p + "att.o_proj.weight"])
            h = P.plain_rmsnorm(x, Wd[p + "ln2.weight"], 1e-6)
            x = x + P.plain_mlp(h, Wd[p + "ffn.gate_proj.weight"], Wd[p + "ffn.up_proj.weight"], Wd[p + "ffn.down_proj.weight"], 1.0)
        return 3.0 * torch.tanh(P.plain_linear(P.plain_rmsnorm(x, Wd["ln_f.weight"], 1e-6), Wd["emb.weight"], None, 0.5) / 3.0)

    drv = Driver(mdir, "float32", num_pages=16, page_size=8, max_requests=2)
    assert drv.model.head_is_tied and type(drv.model.output_head).__name__ == "ToyCappedHead"
    g2 = torch.Generator().manual_seed(5)
    a, b = (torch.randint(0, V, (n,), generator=g2).tolist() for n in (61, 18))
    drv.step([("a", a[:30])])
    drv.step([("a", a[30:32]), ("b", b)], end=["b"])
    drv.step([("a", a[32:33])])
    drv.step([("a", a[33:])], end=["a"])
    assert rel_err(drv.request_logits("a", 61), plain(a)) < 1e-4
    assert rel_err(drv.request_logits("b", 18), plain(b)) < 1e-4
    with pytest.raises(ValueError, match="beyond the position encoding"):
        drv.runner.cache.admit("c")
        from infinilm_amd.engine.step import StepEntry
        drv.runner.model.spec.max_positions = 1000   # the model's own bound lifted: the encoding's must hold
        drv.runner.step([StepEntry("c", [1] * (MAXP + 1), [])])


def test_positions_over_two_axes_reach_a_position_encoding(tmp_path):
    """A model whose spec says two position axes: the step carries [2, T] positions (every axis the place in the
    sequence unless an entry brings its own), and a toy encoding defined here adds one learned table by axis 0 and
    another by axis 1 to q and k.  Portions and decoded tokens of two requests, with columns that restart every
    five tokens, against the plain formulas; the cache and the attention keep counting by the place in the sequence."""
    from safetensors.torch import save_file
    from infinilm_amd import kernels
    from infinilm_amd.config import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinilm_amd.engine.loading import build_model, load_model, make_runner
    from infinilm_amd.engine.step import StepEntry
    from infinilm_amd.parts import Param, PositionEncoding, register_position_encoding

    @register_position_encoding("toy_two_axes")
    class ToyTwoAxes(PositionEncoding):
        def __init__(self, head_dim, max_positions, ctx):
            self.head_dim, self.max_positions = int(head_dim), int(max_positions)
            self.rows = torch.empty((self.max_positions, self.head_dim), dtype=ctx.dtype, device=ctx.device)
            self.cols = torch.empty((8, self.head_dim), dtype=ctx.dtype, device=ctx.device)
            self._none = torch.zeros((1, 0), dtype=torch.float32, device=ctx.device)

        def named_parameters(self):
            return {"rows.weight": Param(self.rows), "cols.weight": Param(self.cols)}

        def encode_and_store(self, qkv, batch, view, nh, nkv, d):
            assert batch.position_axes.shape == (2, qkv.shape[0])
            add = self.rows[batch.position_axes[0].long()] + self.cols[batch.position_axes[1].long()]
            qkv[:, :(nh + nkv) * d].view(-1, nh + nkv, d).add_(add[:, None, :])
            kernels.rope_kvwrite(qkv, batch.positions, self._none, self._none, view.k, view.v, view.slots, nh, nkv, d, 0)

    H, d, nh, nkv, V, MAXP = 32, 16, 2, 1, 41, 64

    def build_spec(cfg):
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-6})
        pos = PartSpec("toy_two_axes", {"head_dim": d, "max_positions": MAXP})
        att = PartSpec("gqa_attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "qkv_bias": False,
                                         "out_bias": False, "scale": d ** -0.5, "window": 0, "position": pos})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 24, "bias": False})
        names = {"norm1": "ln1", "mixer": "att", "norm2": "ln2", "ffn": "ffn"}
        layers = [LayerSpec("l.0", "pre_norm", {"norm1": norm, "mixer": att, "norm2": norm, "ffn": ffn}, names, 1.0)]
        return ModelSpec("ToyTwoAxesLM", V, H, MAXP, "emb", 1.0, layers, [LayerRun(0, 0)], norm, "ln_f", HeadSpec("head", 1.0, True),
                         position_axes=2)

    register_architecture(["ToyTwoAxesLM"], dict, build_spec)
    mdir = str(tmp_path / "two_axes")
    os.makedirs(mdir)
    json.dump({"architectures": ["ToyTwoAxesLM"], "torch_dtype": "float32"}, open(os.path.join(mdir, "config.json"), "w"))
    names = build_model({"architectures": ["ToyTwoAxesLM"]}, "float32", "meta").named_parameters()
    g = torch.Generator().manual_seed(21)
    W = {}
    for name, p in sorted(names.items()):
        if name == "head.weight":
            continue
        t = torch.randn(tuple(p.tensor.shape), generator=g) * 0.4
        W[name] = (t * 0.25 + 1.0) if t.dim() == 1 else t
    save_file(W, os.path.join(mdir, "model.safetensors"), metadata={"format": "pt"})
    col = lambda i: i % 5

    def plain(ids):
        Wd = {k: v.to(F64) for k, v in W.items()}
        n = len(ids)
        x = Wd["emb.weight"][torch.tensor(ids)]
        h = P.plain_rmsnorm(x, Wd["l.0.ln1.weight"], 1e-6)
        off = (Wd["l.0.att.position.rows.weight"][:n] + Wd["l.0.att.position.cols.weight"][[col(i) for i in range(n)]])[:, None, :]
        q = P.plain_linear(h, Wd["l.0.att.q_proj.weight"]).view(n, nh, d) + off
        k = P.plain_linear(h, Wd["l.0.att.k_proj.weight"]).view(n, nkv, d) + off
        v = P.plain_linear(h, Wd["l.0.att.v_proj.weight"]).view(n, nkv, d)
        x = x + P.plain_linear(P.plain_attention(q, k, v, d ** -0.5).reshape(n, nh * d), Wd["l.0.att.o_proj.weight"])
        h = P.plain_rmsnorm(x, Wd["l.0.ln2.weight"], 1e-6)
        x = x + P.plain_mlp(h, Wd["l.0.ffn.gate_proj.weight"], Wd["l.0.ffn.up_proj.weight"], Wd["l.0.ffn.down_proj.weight"], 1.0)
        return P.plain_linear(P.plain_rmsnorm(x, Wd["ln_f.weight"], 1e-6), Wd["emb.weight"])

    model = load_model(mdir, "float32", "cuda:0")
    r = make_runner(model, num_pages=12, page_size=8, max_requests=2)
    g2 = torch.Generator().manual_seed(6)
    a, b = (torch.randint(0, V, (n,), generator=g2).tolist() for n in (40, 13))
    got = {"a": [], "b": []}

    def step(parts):
        es = []
        for rid, toks, lo in parts:
            if not r.cache.has(rid):
                r.cache.admit(rid)
            idx = list(range(lo, lo + len(toks)))
            es.append(StepEntry(rid, toks, list(range(len(toks))), positions=[idx, [col(i) for i in idx]]))
        out = r.step(es).cpu()
        row = 0
        for rid, toks, _ in parts:
            got[rid].append(out[row:row + len(toks)].clone())
            row += len(toks)

    step([("a", a[:17], 0)])
    step([("a", a[17:19], 17), ("b", b, 0)])
    step([("a", a[19:20], 19)])
    step([("a", a[20:], 20)])
    assert rel_err(torch.cat(got["a"]), plain(a)) < 1e-4
    assert rel_err(torch.cat(got["b"]), plain(b)) < 1e-4
    with pytest.raises(ValueError, match=r"positions must be \[2\]"):
        r.step([StepEntry("a", [1], [0], positions=[[40]])])


def test_a_model_without_paged_keys_runs_through_the_entry_point_with_graphs(tmp_path):
    """Every mixer keeps a fixed-size state and none keeps pages: the scheduler's worst-case
    admission, the recorded decode steps and the look-ahead loop have no block table to lean on."""
    from safetensors.torch import save_file
    from infinilm_amd import LLM, SamplingParams
    from infinilm_amd.config import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinilm_amd.engine.loading import build_model

    _register_toy()   # the toy mixer

    def build_spec(cfg):
        H = cfg["hidden_size"]
        norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
        toy = PartSpec("toy_decay", {"hidden_size": H, "state_size": 20, "decay": 0.8})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": 48, "bias": False})
        names = {"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "ffn": "ffn"}
        layers = [LayerSpec(f"b.{i}", "pre_norm", {"norm1": norm, "mixer": toy, "norm2": norm, "ffn": ffn}, names, 0.7) for i in range(2)]
        return ModelSpec("ToyStateOnlyLM", cfg["vocab_size"], H, 512, "emb", 1.0, layers, [LayerRun(0, 0), LayerRun(1, 1)], norm,
                         "ln_f", HeadSpec("head", 1.0, True))

    register_architecture(["ToyStateOnlyLM"], dict, build_spec)
    cfg = {"architectures": ["ToyStateOnlyLM"], "torch_dtype": "float32", "vocab_size": 71, "hidden_size": 32}
    mdir = str(tmp_path / "state_only")
    os.makedirs(mdir)
    json.dump(cfg, open(os.path.join(mdir, "config.json"), "w"))
    g = torch.Generator().manual_seed(2)
    W = {}
    for name, p in sorted(build_model(cfg, "float32", "meta").named_parameters().items()):
        if name == "head.weight":
            continue
        t = torch.randn(tuple(p.tensor.shape), generator=g) * 0.4
        W[name] = (t * 0.25 + 1.0) if t.dim() == 1 else t
    save_file(W, os.path.join(mdir, "model.safetensors"), metadata={"format": "pt"})

    def plain_logits(ids):
        Wd = {k: v.to(F64) for k, v in W.items()}
        x = Wd["emb.weight"][torch.tensor(ids)]
        for l in range(2):
            p = f"b.{l}."
            h = P.plain_rmsnorm(x, Wd[p + "ln1.weight"], 1e-5)
            u = h @ Wd[p + "mix.in_proj.weight"].T
            s, rows = torch.zeros(20, dtype=F64), []
            for t in range(len(ids)):
                s = 0.8 * s + u[t]
                rows.append(s)
            x = x + 0.7 * (torch.stack(rows) @ Wd[p + "mix.out_proj.weight"].T)
            h = P.plain_rmsnorm(x, Wd[p + "ln2.weight"], 1e-5)
            x = x + 0.7 * P.plain_mlp(h, Wd[p + "ffn.gate_proj.weight"], Wd[p + "ffn.up_proj.weight"], Wd[p + "ffn.down_proj.weight"], 1.0)
        return P.plain_linear(P.plain_rmsnorm(x, Wd["ln_f.weight"], 1e-5), Wd["emb.weight"])

    def plain_greedy(ids, n):
        ids, out = list(ids), []
        for _ in range(n):
            out.append(int(torch.argmax(plain_logits(ids)[-1])))
            ids.append(out[-1])
        return out

    g2 = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 71, (n,), generator=g2).tolist() for n in (9, 1, 23, 14)]
    for policy in ("reserve_full", "optimistic"):
        # (the second time with every decode step size recorded before the first request: three requests
        # at most, no pages: the sizes 1, 2 and 4)
        at_start = policy == "optimistic"
        llm = LLM(mdir, dtype="float32", num_blocks=4, block_size=16, max_batch_size=3, chunk_size=8, max_num_batched_tokens=16,
                  enable_graph=True, admission=policy, record_graphs_at_start=at_start)
        assert not llm.engine.runner.cache.groups
        assert len(llm.engine.runner._graphs) == (3 if at_start else 0)
        outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(top_k=1, max_tokens=12, ignore_eos=True))
        for p, o in zip(prompts, outs):
            assert o.outputs[0].token_ids == plain_greedy(p, 12), f"{policy}: prompt of {len(p)} tokens"
        assert llm.engine.runner._graphs, "no decode step was recorded"
        assert not at_start or len(llm.engine.runner._graphs) == 3
        llm.engine.runner.cache.check()
        llm.close()
