"""The products of a decode step with both operands in fragment order (csrc/frag.h, csrc/gemm_frag.hip): the
packers, the plain product in its four result forms, and the three fused epilogues, each against the plain
formulas in float64, at sizes that are no multiple of a tile, a k-step or a row group."""
import math

import pytest
import torch

import plain_minicpm4 as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
BF = torch.bfloat16


@pytest.fixture(scope="module")
def K():
    from infinilm_amd import kernels
    return kernels


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(BF)


def _close(got, want, tol):
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    err = float((got - want).abs().max() / max(1.0, float(want.abs().max())))
    assert err < tol, f"error {err:.3e} above {tol:.1e}"


@pytest.mark.parametrize("M,Kd", [(1, 8), (5, 96), (16, 4096), (17, 200), (64, 1032), (33, 40)])
def test_rows_into_fragment_order_and_back(K, M, Kd):
    x = _rand((M, Kd), 1)
    f = K.to_frag(x.to(DEV))
    assert torch.equal(K.from_frag(f).cpu(), x)
    # the layout itself: lane (r, q) of group g, step s holds row 16 g + r, k 32 s + 8 q ..
    raw = f.data.view(torch.bfloat16).view(-(-Kd // 32), -(-M // 16), 4, 16, 8).cpu()
    for m, k in ((0, 0), (M - 1, Kd - 8), (M // 2, (Kd // 16) * 8)):
        assert torch.equal(raw[k // 32, m // 16, (k % 32) // 8, m % 16], x[m, k:k + 8])
    if Kd % 32:
        assert not raw[-1, :, (Kd % 32) // 8:].any(), "k beyond the width must be zeros"


@pytest.mark.parametrize("M,N,Kd,bias", [(1, 16, 32, False), (5, 331, 80, True), (16, 4608, 4096, False), (17, 96, 200, True),
                                         (64, 50, 1032, False), (33, 4096, 4096, False), (48, 200, 16384, True),
                                         (8, 73448, 1024, False)])
@pytest.mark.parametrize("tiles", [2, 4])
def test_plain_product(K, monkeypatch, M, N, Kd, bias, tiles):
    monkeypatch.setattr(K, "FRAG_TILES", tiles)
    x, w = _rand((M, Kd), 2), _rand((N, Kd), 3, Kd ** -0.5)
    b = _rand((N,), 4) if bias else None
    fw = K.pack_weight(w.to(DEV))
    fx = K.to_frag(x.to(DEV))
    want = P.plain_linear(x.to(F64), w.to(F64), None if b is None else b.to(F64), 0.5)
    dev = lambda t: None if t is None else t.to(DEV)
    _close(K.gemm_frag(fx, fw, dev(b), 0.5, out="f32"), want, 1e-5 * math.sqrt(Kd) + 2e-6)
    _close(K.gemm_frag(fx, fw, dev(b), 0.5, out="bf16"), want, 6e-3)
    if N % 8 == 0:   # (a result in fragment order feeds a product over it: widths are multiples of 8 there)
        _close(K.from_frag(K.gemm_frag(fx, fw, dev(b), 0.5, out="frag")), want, 6e-3)
    for parts in (2, 4, 16):
        p = K.gemm_frag(fx, fw, dev(b), 0.5, out="parts", parts=parts)
        assert p.shape[0] <= parts and p.shape[1:] == (M, N)
        _close(p.sum(0), want, 1e-5 * math.sqrt(Kd) + 2e-6)
    # a row does not depend on the rows around it, bit for bit, whatever their number
    full = K.gemm_frag(fx, fw, dev(b), 0.5, out="f32").cpu()
    one = K.gemm_frag(K.to_frag(x[M // 2:M // 2 + 1].to(DEV)), fw, dev(b), 0.5, out="f32").cpu()
    assert torch.equal(one[0], full[M // 2])


@pytest.mark.parametrize("M,I,Kd,bias", [(8, 16384, 4096, False), (3, 200, 96, True), (17, 328, 1032, True), (64, 4104, 256, False),
                                         (40, 24, 40, True)])
@pytest.mark.parametrize("tiles", [2, 4])
def test_gate_up_with_the_activation_in_the_epilogue(K, monkeypatch, M, I, Kd, bias, tiles):
    monkeypatch.setattr(K, "FRAG_TILES", tiles)
    x, w = _rand((M, Kd), 5), _rand((2 * I, Kd), 6, Kd ** -0.5)
    b = _rand((2 * I,), 7) if bias else None
    fw = K.pack_weight(w.to(DEV), "gate_up")
    act = K.gemm_frag_swiglu(K.to_frag(x.to(DEV)), fw, None if b is None else b.to(DEV))
    y = P.plain_linear(x.to(F64), w.to(F64), None if b is None else b.to(F64))
    _close(K.from_frag(act), P.plain_swiglu(y[:, :I], y[:, I:]), 1.5e-2)
    if I % 32:
        raw = act.data.view(torch.bfloat16).view(-(-I // 32), -(-M // 16), 4, 16, 8).cpu()
        assert not raw[-1, :, -(-(I % 32) // 8):].any()


@pytest.mark.parametrize("M,nh,nkv,d,Kd,page,bias", [(5, 4, 2, 32, 96, 8, False), (16, 32, 2, 128, 4096, 64, False),
                                                     (1, 3, 3, 64, 200, 16, True), (64, 32, 2, 128, 4096, 64, False),
                                                     (33, 4, 2, 32, 96, 8, True), (40, 3, 3, 96, 8200, 16, True),
                                                     (57, 36, 36, 64, 2304, 16, False)])
def test_qkv_projection_with_rotation_and_cache_write(K, M, nh, nkv, d, Kd, page, bias):
    max_pos = 300
    N = (nh + 2 * nkv) * d
    x, w = _rand((M, Kd), 21), _rand((N, Kd), 22, Kd ** -0.5)
    b = _rand((N,), 23) if bias else None
    g = torch.Generator().manual_seed(24)
    pos = torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32)
    pos[0] = max_pos - 1
    cfg = {"hidden_size": d, "num_attention_heads": 1, "max_position_embeddings": max_pos, "rope_theta": 5000.0}
    cos, sin = P.plain_rope_tables(cfg)
    n_pages = M + 2
    slots = (torch.randperm(n_pages, generator=g)[:M] * page + torch.randint(0, page, (M,), generator=g)).to(torch.int32)
    if M > 2:
        slots[2] = -1   # a token that is not cached
    dev = lambda t: None if t is None else t.to(DEV)
    kc = torch.zeros((n_pages, nkv, page, d), dtype=BF, device=DEV)
    vc = torch.zeros((n_pages, nkv, d, page), dtype=BF, device=DEV)
    fw = K.pack_weight(dev(w), "qkv", nh=nh, nkv=nkv, d=d)
    q = K.gemm_frag_rope(K.to_frag(dev(x)), fw, dev(b), dev(pos), dev(cos.float()), dev(sin.float()), kc, vc, dev(slots), nh, nkv, d)
    y = P.plain_linear(x.to(F64), w.to(F64), None if b is None else b.to(F64)).view(M, nh + 2 * nkv, d)
    _close(q, P.plain_apply_rope(y[:, :nh], pos, cos, sin, d).reshape(M, nh * d), 1e-2)
    want_k = P.plain_apply_rope(y[:, nh:nh + nkv], pos, cos, sin, d)
    kc, vc = kc.cpu().float(), vc.cpu().float()
    written = torch.zeros(n_pages * page, dtype=torch.bool)
    for t in range(M):
        s = int(slots[t])
        if s < 0:
            continue
        written[s] = True
        _close(kc[s // page, :, s % page, :], want_k[t], 1e-2)
        _close(vc[s // page, :, :, s % page], y[t, nh + nkv:], 1e-2)
    untouched = ~written.view(n_pages, page)
    assert not kc.permute(0, 2, 1, 3)[untouched].any() and not vc.permute(0, 3, 1, 2)[untouched].any()


@pytest.mark.parametrize("M,Ko,H,I,bias,wdt", [(8, 4096, 4096, 16384, False, BF), (3, 96, 80, 200, True, torch.float32),
                                               (64, 1024, 1024, 4096, False, BF), (17, 136, 72, 40, True, BF), (33, 256, 2304, 64, False, BF)])
@pytest.mark.parametrize("tiles", [2, 4])
def test_branch_tail_and_the_norm_finished_by_the_gate_up_product(K, monkeypatch, M, Ko, H, I, bias, wdt, tiles):
    """o projection with the residual sum and half of the following norm in its epilogue, then the gate/up product
    that finishes the norm: against add, RMS norm, projection and SwiGLU in float64."""
    monkeypatch.setattr(K, "FRAG_TILES", tiles)
    eps, alpha = 1e-5, 0.37
    x, wo = _rand((M, Ko), 31), _rand((H, Ko), 32, Ko ** -0.5)
    bo = _rand((H,), 33) if bias else None
    r0 = torch.randn((M, H), generator=torch.Generator().manual_seed(34))
    nw = (1.0 + 0.1 * torch.randn((H,), generator=torch.Generator().manual_seed(35))).to(wdt)
    wgu = _rand((2 * I, H), 36, H ** -0.5)
    dev = lambda t: None if t is None else t.to(DEV)
    r = r0.clone().to(DEV)
    xw, ss = K.gemm_frag_tail(K.to_frag(dev(x)), K.pack_weight(dev(wo)), dev(bo), alpha, r, dev(nw))
    want_r = r0.to(F64) + alpha * P.plain_linear(x.to(F64), wo.to(F64), None if bo is None else bo.to(F64))
    _close(r, want_r, 1e-5 * math.sqrt(Ko) + 2e-6)
    _close(K.from_frag(xw), want_r * nw.to(F64), 6e-3)
    got_ss = ss.to(F64).sum(0)[:M].cpu()
    assert float(((got_ss - (want_r ** 2).sum(1)).abs() / (want_r ** 2).sum(1)).max()) < 1e-5
    act = K.gemm_frag_swiglu(xw, K.pack_weight(dev(wgu), "gate_up"), None, row_ss=ss, norm_width=H, eps=eps)
    h = P.plain_rmsnorm(want_r, nw.to(F64), eps)
    y = P.plain_linear(h, wgu.to(F64), None)
    _close(K.from_frag(act), P.plain_swiglu(y[:, :I], y[:, I:]), 2e-2)
