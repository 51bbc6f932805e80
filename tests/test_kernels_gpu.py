"""Each HIP kernel alone against a plain PyTorch float64 reference of the same op, at other sizes
than the engine tests use: odd widths, head sizes in steps of 16, groups of 1 to 16 heads, contexts
that cross pages and key chunks, a far key that must dominate, a window's edge."""
import math

import pytest
import torch

import plain_minicpm4 as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


@pytest.fixture(scope="module")
def K():
    from infinilm_amd import kernels
    return kernels


def _rand(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _close(got, want, tol):
    got = got.detach().cpu().to(F64)
    want = want.detach().cpu().to(F64)
    err = float((got - want).abs().max() / max(1.0, float(want.abs().max())))
    assert err < tol, f"error {err:.3e} above {tol:.1e}"


def test_constants_mirrored_in_python_equal_the_library(K):
    from infinilm_amd.csrc import lib
    L = lib.load()
    assert L.ilm_attn_tile_tokens() == K.ATT_TILE_TOKENS
    assert L.ilm_attn_mfma_step() == K.ATT_STEP
    assert L.ilm_attn_basic_chunk() == K.BASIC_CHUNK
    assert L.ilm_attn_f32_chunk() == K.F32_ATTN_CHUNK and L.ilm_attn_f32_ws_row(128) == 132
    assert L.ilm_gemm_ksplit_max_k(1) == K.KSPLIT_SPAN
    assert L.ilm_gemm_rows64_span() == K.ROWS64_SPAN


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(K, dtype):
    table = _rand((331, 80), 1, dtype)
    ids = torch.tensor([0, 330, 7, 7, 100], dtype=torch.int32)
    out = K.embed(ids.to(DEV), table.to(DEV), 7.5)
    assert out.dtype == torch.float32
    _close(out, table.to(F64)[ids.long()] * 7.5, 1e-6)


@pytest.mark.parametrize("dtype,wdtype,H", [(torch.float32, torch.float32, 80), (torch.bfloat16, torch.bfloat16, 331),
                                            (torch.bfloat16, torch.float32, 4096), (torch.float32, torch.float32, 1)])
def test_add_rmsnorm(K, dtype, wdtype, H):
    r = _rand((5, H), 2, scale=3.0)
    h = _rand((5, H), 3, dtype)
    w = _rand((H,), 4, wdtype) + 1
    rd = r.to(DEV).clone()
    x = K.add_rmsnorm(rd, h.to(DEV), w.to(DEV), 0.37, 1e-5, dtype)
    want_r = r.to(F64) + 0.37 * h.to(F64)
    _close(rd, want_r, 1e-6)
    want = P.plain_rmsnorm(want_r, w.to(F64), 1e-5)
    _close(x, want, 2e-6 if dtype == torch.float32 else 1e-2)
    # without a branch the residual is untouched
    rd2 = r.to(DEV).clone()
    x2 = K.add_rmsnorm(rd2, None, w.to(DEV), 1.0, 1e-5, dtype)
    assert torch.equal(rd2.cpu(), r)
    _close(x2, P.plain_rmsnorm(r.to(F64), w.to(F64), 1e-5), 2e-6 if dtype == torch.float32 else 1e-2)
    # a row's result does not depend on the batch around it
    x1 = K.add_rmsnorm(r[2:3].to(DEV).clone(), None, w.to(DEV), 1.0, 1e-5, dtype)
    assert torch.equal(x1.cpu(), x2[2:3].cpu())


@pytest.mark.parametrize("rows,H,parts,wdtype", [(64, 4096, 16, torch.bfloat16), (33, 2304, 4, torch.float32), (5, 72, 7, torch.bfloat16),
                                                 (208, 1032, 9, torch.bfloat16), (17, 4096, 3, torch.bfloat16), (40, 4104, 8, torch.bfloat16)])
def test_add_rmsnorm_of_few_rows_with_many_float_parts(K, rows, H, parts, wdtype):
    """The float32 parts of a K-split product into bfloat16 activations: 4 to 16 parts of rows up to 4096 wide take the
    kernel with 16 waves a row (3 parts, or a wider row, the general one); plain rows and fragment order; the same
    row gives the same bits whatever the rows around it."""
    r = _rand((rows, H), 2, scale=3.0)
    h = _rand((parts, rows, H), 3, scale=0.5)
    w = _rand((H,), 4, wdtype) + 1
    want_r = r.to(F64) + 0.37 * h.to(F64).sum(0)
    want = P.plain_rmsnorm(want_r, w.to(F64), 1e-5)
    rd = r.to(DEV).clone()
    x = K.add_rmsnorm(rd, h.to(DEV), w.to(DEV), 0.37, 1e-5, torch.bfloat16)
    _close(rd, want_r, 1e-6)
    _close(x, want, 1e-2)
    if rows <= K.FRAG_MAX_ROWS:
        rd2 = r.to(DEV).clone()
        xf = K.add_rmsnorm(rd2, h.to(DEV), w.to(DEV), 0.37, 1e-5, torch.bfloat16, frag=True)
        assert torch.equal(rd2, rd) and torch.equal(K.from_frag(xf), x)
        if H % 32:   # the k up to the next multiple of 32 are zeros in fragment order
            raw = xf.data.view(torch.bfloat16).view(-(-H // 32), -(-rows // 16), 4, 16, 8).cpu()
            assert not raw[-1, :, (H % 32) // 8:].any()
    one = K.add_rmsnorm(r[3:4].to(DEV).clone(), h[:, 3:4].contiguous().to(DEV), w.to(DEV), 0.37, 1e-5, torch.bfloat16)
    assert torch.equal(one, x[3:4])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,rd,page", [(4, 2, 16, 16, 4), (3, 1, 48, 48, 16), (5, 5, 32, 16, 8), (2, 1, 80, 0, 16)])
def test_rope_and_cache_write(K, dtype, nh, nkv, d, rd, page):
    T, max_pos = 9, 50
    qkv = _rand((T, (nh + 2 * nkv) * d), 5, dtype)
    pos = torch.tensor([0, 1, 2, 17, 49, 3, 3, 30, 11], dtype=torch.int32)
    cfg = {"hidden_size": d, "num_attention_heads": 1, "max_position_embeddings": max_pos, "rope_theta": 777.0,
           "partial_rotary_factor": rd / d if 0 < rd < d else 1.0}
    if rd > 0:
        cos, sin = P.plain_rope_tables(cfg)
    else:
        cos, sin = torch.zeros(max_pos, 0, dtype=F64), torch.zeros(max_pos, 0, dtype=F64)
    n_pages = 7
    kc = torch.zeros((n_pages, nkv, page, d), dtype=dtype, device=DEV)
    vc = torch.zeros((n_pages, nkv, d, page), dtype=dtype, device=DEV)
    slots = torch.tensor([5 * page + 1, 0, 2 * page + page - 1, -1, 6 * page, 3 * page + 2, page, page + 1, 4 * page],
                         dtype=torch.int32)
    buf = qkv.to(DEV).clone()
    K.rope_kvwrite(buf, pos.to(DEV), cos.float().to(DEV), sin.float().to(DEV), kc, vc, slots.to(DEV), nh, nkv, d, rd)
    x = qkv.to(F64).view(T, nh + 2 * nkv, d)
    want_q = P.plain_apply_rope(x[:, :nh], pos, cos, sin, rd) if rd else x[:, :nh]
    want_k = P.plain_apply_rope(x[:, nh:nh + nkv], pos, cos, sin, rd) if rd else x[:, nh:nh + nkv]
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    got = buf.cpu().view(T, nh + 2 * nkv, d)
    _close(got[:, :nh], want_q, tol)
    _close(got[:, nh:nh + nkv], want_k, tol)
    assert torch.equal(got[:, nh + nkv:], qkv.view(T, nh + 2 * nkv, d)[:, nh + nkv:])   # v untouched
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        pg, off = s // page, s % page
        assert torch.equal(kc[pg, :, off, :].cpu(), got[t, nh:nh + nkv])        # the rotated key is what is cached
        assert torch.equal(vc[pg, :, :, off].cpu(), got[t, nh + nkv:])           # values lie transposed
    written = {int(s) for s in slots if s >= 0}
    mask = torch.ones(n_pages * page, dtype=torch.bool)
    mask[list(written)] = False
    assert not kc.cpu().permute(0, 2, 1, 3).reshape(n_pages * page, -1)[mask].any()  # nothing else was touched


@pytest.mark.parametrize("M,nh,nkv,d,Kd,page,bias", [(5, 4, 2, 32, 96, 8, False), (16, 32, 2, 128, 4096, 64, False),
                                                     (1, 3, 3, 64, 200, 16, True), (8, 16, 2, 64, 1024, 16, False),
                                                     (3, 2, 1, 96, 8192, 4, True), (17, 4, 2, 32, 96, 8, True),
                                                     (32, 32, 2, 128, 4096, 64, False), (24, 16, 2, 64, 1024, 16, False),
                                                     (29, 3, 3, 96, 2056, 16, True)])
def test_projection_with_rotation_and_cache_write_in_one_kernel(K, M, nh, nkv, d, Kd, page, bias):
    """The decode-side fused kernel against the plain product + rotation, and against the
    product kernel followed by the rotation kernel."""
    max_pos = 300
    N = (nh + 2 * nkv) * d
    x, w = _rand((M, Kd), 21, torch.bfloat16), _rand((N, Kd), 22, torch.bfloat16, scale=Kd ** -0.5)
    b = _rand((N,), 23, torch.bfloat16) if bias else None
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
    caches = []
    for fused in (True, False):
        kc = torch.zeros((n_pages, nkv, page, d), dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros((n_pages, nkv, d, page), dtype=torch.bfloat16, device=DEV)
        if fused:
            q = K.qkv_rope_gemm(dev(x), dev(w), dev(b), dev(pos), dev(cos.float()), dev(sin.float()), kc, vc, dev(slots),
                                nh, nkv, d, d)
            assert q is not None
        else:
            qkv = K.gemm(dev(x), dev(w), dev(b))
            K.rope_kvwrite(qkv, dev(pos), dev(cos.float()), dev(sin.float()), kc, vc, dev(slots), nh, nkv, d, d)
            q = qkv[:, :nh * d]
        caches.append((q.cpu().float(), kc.cpu().float(), vc.cpu().float()))
    y = P.plain_linear(x.to(F64), w.to(F64), None if b is None else b.to(F64)).view(M, nh + 2 * nkv, d)
    want_q = P.plain_apply_rope(y[:, :nh], pos, cos, sin, d).reshape(M, nh * d)
    want_k = P.plain_apply_rope(y[:, nh:nh + nkv], pos, cos, sin, d)
    q, kc, vc = caches[0]
    _close(q, want_q, 1e-2)
    for t in range(M):
        s = int(slots[t])
        if s < 0:
            continue
        _close(kc[s // page, :, s % page, :], want_k[t], 1e-2)
        _close(vc[s // page, :, :, s % page], y[t, nh + nkv:], 1e-2)
    # the two paths round the projection to bfloat16 at the same place: they agree to an ulp of the result
    for a, b_ in zip(caches[0], caches[1]):
        assert (a - b_).abs().max() <= 2 ** -7 * max(a.abs().max(), 1e-6)
        assert ((a != 0) == (b_ != 0)).all()   # and write the same places, nothing else


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_and_gather(K, dtype):
    gu = _rand((7, 2 * 200), 6, dtype, 2.0)
    out = K.swiglu(gu.to(DEV))
    g, u = gu.to(F64)[:, :200], gu.to(F64)[:, 200:]
    _close(out, P.plain_swiglu(g, u), 2e-6 if dtype == torch.float32 else 1e-2)
    x = _rand((11, 96), 7, dtype)
    idx = torch.tensor([10, 0, 3, 3], dtype=torch.int32)
    assert torch.equal(K.gather_rows(x.to(DEV), idx.to(DEV)).cpu(), x[idx.long()])


@pytest.mark.parametrize("M,N,K_", [(1, 1, 1), (5, 331, 80), (64, 96, 200), (130, 70, 33), (3, 4608, 4096), (17, 331, 4100),
                                    (33, 50, 12296), (48, 4608, 1032), (8, 16400, 64), (20, 32768, 256), (200, 96, 200),
                                    (65, 130, 4), (300, 1100, 1028), (129, 257, 44), (2048, 1024, 4096)])
def test_gemm_float32_is_true_float32(K, M, N, K_):
    a, w, b = _rand((M, K_), 8), _rand((N, K_), 9), _rand((N,), 10)
    out = K.gemm(a.to(DEV), w.to(DEV), b.to(DEV), 0.25)
    want = P.plain_linear(a.to(F64), w.to(F64), b.to(F64), 0.25)
    _close(out, want, 2e-6 * math.sqrt(K_))   # no reduced-precision matrix mode: errors of float32 sums only
    # Rows do not depend on the batch around them, bit for bit: the few-rows kernel (up to 64 rows) and the tile
    # kernel (more) sum every output in one order, fixed by K alone (as does the plain ascending-k kernel, which
    # takes every row count of a K that is no multiple of 4).
    one = K.gemm(a[M // 2:M // 2 + 1].to(DEV), w.to(DEV), b.to(DEV), 0.25)
    assert torch.equal(one.cpu(), out[M // 2:M // 2 + 1].cpu())
    some = K.gemm(a[:min(M, 3)].to(DEV), w.to(DEV), b.to(DEV), 0.25)
    assert torch.equal(some.cpu(), out[:min(M, 3)].cpu())
    more = K.gemm(torch.cat([a, a[:70]]).to(DEV), w.to(DEV), b.to(DEV), 0.25)
    assert torch.equal(more[:M].cpu(), out.cpu())


@pytest.mark.parametrize("M,N,K_,out_dtype", [
    (1, 16, 32, torch.bfloat16), (1, 4608, 4096, torch.bfloat16), (8, 331, 80, torch.float32), (17, 96, 200, torch.bfloat16),
    (33, 200, 96, torch.bfloat16), (64, 73448, 128, torch.float32), (48, 100, 2048, torch.bfloat16),
    (7, 50, 100, torch.bfloat16),        # K no multiple of 8: the plain kernel takes it
    (100, 176, 80, torch.bfloat16), (300, 512, 256, torch.bfloat16), (65, 40, 64, torch.float32), (40, 331, 96, torch.float32),
    (32, 4608, 4096, torch.bfloat16), (25, 331, 4096, torch.float32), (20, 100, 1032, torch.bfloat16),   # two row groups in registers
    (31, 50, 4104, torch.bfloat16),      # K beyond what two row groups hold: the library
])
def test_gemm_bfloat16(K, M, N, K_, out_dtype):
    a, w = _rand((M, K_), 11, torch.bfloat16), _rand((N, K_), 12, torch.bfloat16)
    alpha = 0.3 if out_dtype == torch.float32 else 1.0
    out = K.gemm(a.to(DEV), w.to(DEV), None, alpha, out_dtype)
    assert out.dtype == out_dtype
    want = P.plain_linear(a.to(F64), w.to(F64), None, alpha)
    _close(out, want, 1e-5 if out_dtype == torch.float32 else 6e-3)
    if M <= 64:
        b = _rand((N,), 13, torch.bfloat16)
        out = K.gemm(a.to(DEV), w.to(DEV), b.to(DEV), 0.5, out_dtype)
        _close(out, P.plain_linear(a.to(F64), w.to(F64), b.to(F64), 0.5), 1e-5 if out_dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("M,N,K_", [(8, 4096, 16384), (1, 50, 8200), (16, 331, 12296), (17, 4096, 4096), (64, 4096, 16384),
                                    (48, 331, 200), (35, 50, 8200), (128, 1030, 1096), (97, 64, 72), (32, 4096, 16384),
                                    (20, 331, 12296), (27, 50, 8200), (5, 96, 5760), (30, 2304, 5760), (192, 4096, 16384), (208, 331, 4096),
                                    (150, 331, 1096), (177, 96, 200)])
@pytest.mark.parametrize("tall", [True, False])
def test_gemm_split_over_k_and_its_consumer(K, monkeypatch, M, N, K_, tall):
    """Few rows and long K: the product comes as float32 parts; add_rmsnorm sums them in order.  `tall`: with the
    product that keeps chunks of X in LDS (17 to 208 rows of a matrix that fills the chip), and with the kernels
    that serve when it is switched off."""
    monkeypatch.setattr(K, "USE_TALL", tall)
    a, w = _rand((M, K_), 14, torch.bfloat16), _rand((N, K_), 15, torch.bfloat16, 0.05)
    if M > 64 and not (tall and K._tall_fills_the_chip(N, K_, torch.device(DEV))):
        # many rows of a small matrix (or without that product) are left to the library on the engine's path
        assert K.gemm(a.to(DEV), w.to(DEV), allow_parts=True).dtype == torch.bfloat16
        if not tall:
            return
        monkeypatch.setattr(K, "TALL_MIN_WGS_PER_CU", -1.0)   # the kernel is tested all the same
    parts = K.gemm(a.to(DEV), w.to(DEV), allow_parts=True)
    if tall and 16 < M <= K.TALL_MAX_ROWS and K_ % 8 == 0 and K._tall_fills_the_chip(N, K_, torch.device(DEV)):
        assert parts.shape[0] == K._tall_plan(M, N, K_)[1] <= K.TALL_MAX_PARTS
    elif 16 < M <= 64 and K_ % 8 == 0:   # K ranges of 1024 (up to 32 rows with K beyond 4096: ranges of 4096)
        assert parts.shape[0] == (-(-K_ // 4096) if M <= 32 and K_ > 4096 else -(-K_ // 1024))
    if parts.dim() == 2:   # short K and few rows: one float32 result
        assert K_ <= 4096 and M <= 16
        parts = parts[None]
    assert parts.dim() == 3 and parts.dtype == torch.float32
    assert M > 16 or K_ <= 4096 or parts.shape[0] == -(-K_ // 4096)   # up to 16 rows: K ranges of 4096
    want = P.plain_linear(a.to(F64), w.to(F64))
    _close(parts.sum(0), want, 1e-5)
    whole = K.gemm(a.to(DEV), w.to(DEV))
    assert whole.dim() == 2 and whole.dtype == torch.bfloat16
    short = K.gemm(a[:, :256].contiguous().to(DEV), w[:, :256].contiguous().to(DEV), allow_parts=True)
    # short K: float32, not rounded to bfloat16 (more than 16 rows: parts)
    # (many rows of a small matrix: the library's bfloat16 result)
    assert (short.dtype == torch.float32 and short.dim() == 2) if M <= 16 else (short.dim() == 3 or M > 64)
    _close(whole, want, 6e-3)
    r = _rand((M, N), 16, scale=2.0)
    nw = _rand((N,), 17, torch.bfloat16) + 1
    rd = r.to(DEV).clone()
    x = K.add_rmsnorm(rd, parts, nw.to(DEV), 0.3, 1e-6, torch.bfloat16)
    want_r = r.to(F64) + 0.3 * want
    _close(rd, want_r, 1e-5)
    _close(x, P.plain_rmsnorm(want_r, nw.to(F64), 1e-6), 1e-2)


@pytest.mark.parametrize("M,I,N", [(8, 16384, 4096), (3, 200, 96), (16, 4104, 50), (17, 4104, 50), (32, 16384, 4096),
                                   (24, 200, 96), (33, 96, 331)])
def test_swiglu_inside_the_down_projection(K, M, I, N):
    gu = _rand((M, 2 * I), 18, torch.bfloat16, 1.5)
    w = _rand((N, I), 19, torch.bfloat16, 0.05)
    if M > 32:   # more rows: the activation kernel and a product of its own
        assert K.swiglu_gemm(gu.to(DEV), w.to(DEV)) is None
        return
    parts = K.swiglu_gemm(gu.to(DEV), w.to(DEV))
    assert parts is not None and parts.dtype == torch.float32 and parts.shape[1:] == (M, N)
    assert parts.shape[0] == -(-I // 4096)
    act = P.plain_swiglu(gu.to(F64)[:, :I], gu.to(F64)[:, I:])
    _close(parts.sum(0), P.plain_linear(act, w.to(F64)), 6e-3)   # the activation is rounded to bfloat16 once


@pytest.mark.parametrize("M,I,Kd,bias", [(8, 16384, 4096, False), (3, 200, 96, True), (16, 331, 1032, False), (17, 331, 1032, True),
                                         (32, 4096, 4096, False), (5, 50, 8192, True), (24, 96, 200, False),
                                         (20, 8200, 1032, True), (2, 5760, 2304, False),
                                         # 33 to 64 rows, and 17 to 32 with a long K: chunks of X in LDS
                                         (64, 16384, 4096, False), (33, 331, 1032, True), (48, 200, 96, False), (49, 4100, 520, True),
                                         (40, 5760, 2304, False), (64, 61, 8, True), (20, 96, 8200, False)])
@pytest.mark.parametrize("tall", [False, True])
def test_gate_up_projection_with_the_activation_in_its_epilogue(K, monkeypatch, M, I, Kd, bias, tall):
    """One kernel for silu(x Wg^T) * (x Wu^T) against the plain formula and against the projection
    followed by the activation kernel (gate and up rounded to bfloat16 at the same place).  `tall`: from 17 rows
    the kernel with chunks of X in LDS where the outputs fill the chip; without it the kernel that keeps X in
    registers (up to 32 rows of a K up to 4096)."""
    monkeypatch.setattr(K, "USE_TALL", tall)
    if M > 32 or (M > 16 and Kd > 4096):   # rows that do not fit the registers
        if I < 12288 or not tall:
            # few outputs are left to the library on the engine's path (they do not fill the chip)
            assert K.gateup_swiglu_gemm(_rand((M, Kd), 31, torch.bfloat16).to(DEV), _rand((2 * I, Kd), 32, torch.bfloat16).to(DEV), None) is None
        if not tall:
            return
        monkeypatch.setattr(K, "GATEUP_TALL_MIN_OUTPUTS", 0)   # the kernel is tested all the same
    x, w = _rand((M, Kd), 31, torch.bfloat16), _rand((2 * I, Kd), 32, torch.bfloat16, scale=2.0 * Kd ** -0.5)
    b = _rand((2 * I,), 33, torch.bfloat16) if bias else None
    dev = lambda t: None if t is None else t.to(DEV)
    act = K.gateup_swiglu_gemm(dev(x), dev(w), dev(b))
    assert act is not None and act.shape == (M, I) and act.dtype == torch.bfloat16
    y = P.plain_linear(x.to(F64), w.to(F64), None if b is None else b.to(F64))
    _close(act, P.plain_swiglu(y[:, :I], y[:, I:]), 1e-2)
    two = K.swiglu(K.gemm(dev(x), dev(w), dev(b)))
    assert (act.float() - two.float()).abs().max() <= 2 ** -6 * max(float(two.float().abs().max()), 1e-6)
    assert K.gateup_swiglu_gemm(dev(x.float()), dev(w.float()), None) is None          # float32: not this kernel
    if M <= 32:
        big = _rand((209, Kd), 34, torch.bfloat16)
        assert K.gateup_swiglu_gemm(dev(big), dev(w), dev(b)) is None                  # too many rows


@pytest.mark.parametrize("M,N,K_", [(17, 200, 264), (64, 128, 1024), (65, 334, 520), (100, 4096, 4096), (128, 130, 16384),
                                    (129, 256, 640), (144, 4096, 16384), (208, 512, 2048), (97, 64, 72), (113, 1030, 4104),
                                    (32, 4096, 16384), (48, 2304, 5760)])
def test_products_with_chunks_of_x_in_lds(K, monkeypatch, M, N, K_):
    """`gemm_tall.hip`, both epilogues, chunks of 64 and of 128 k, weights in plain rows and in fragment order, against
    the plain formulas: K no multiple of a chunk, rows and outputs no multiple of a tile, one part and many."""
    from infinilm_amd.csrc import lib
    assert K.TALL_MAX_ROWS == lib.load().ilm_gemm_tall_max_rows()
    x, w = _rand((M, K_), 41, torch.bfloat16), _rand((N, K_), 42, torch.bfloat16, 0.05)
    want = P.plain_linear(x.to(F64), w.to(F64))
    kc, kb, cpp = K._tall_plan(M, N, K_)
    assert kc in (64, 128) and kb <= K.TALL_MAX_PARTS and kb == -(-(-(-K_ // kc)) // cpp)
    other = 192 - kc   # the other chunk length, split into three parts where there are that many chunks
    chunks = -(-K_ // other)
    cpp3 = -(-chunks // 3)
    for plan in ((kc, kb, cpp), (other, -(-chunks // cpp3), cpp3)):
        for fw in (None, K.pack_weight(w.to(DEV))):
            parts = K._gemm_tall(x.to(DEV), w.to(DEV), K_, fw, plan)
            assert parts.dtype == torch.float32 and parts.shape == (plan[1], M, N)
            _close(parts.sum(0), want, 1e-5)
    inter = N // 2
    bias = _rand((2 * inter,), 43, torch.bfloat16, 0.1)
    wg = w[:2 * inter]
    y = P.plain_linear(x.to(F64), wg.to(F64), bias.to(F64))
    want_act = P.plain_swiglu(y[:, :inter], y[:, inter:])
    two = K.swiglu(K.gemm(x.to(DEV), wg.to(DEV), bias.to(DEV)))
    for fw in (None, K.pack_weight(wg.to(DEV), "gate_up8")):
        for b, kc_ in ((bias.to(DEV), 128), (bias.to(DEV), 64), (None, 128)):
            act = K.gemm_tall_swiglu(x.to(DEV), wg.to(DEV), b, fw, kc_)
            assert act.shape == (M, inter) and act.dtype == torch.bfloat16
            if b is None:
                y0 = P.plain_linear(x.to(F64), wg.to(F64))
                _close(act, P.plain_swiglu(y0[:, :inter], y0[:, inter:]), 1e-2)
            else:
                _close(act, want_act, 1e-2)
                # gate and up are rounded to bfloat16 at the same place as the projection followed by the activation kernel
                assert (act.float() - two.float()).abs().max() <= 2 ** -6 * max(float(two.float().abs().max()), 1e-6)


def test_the_plan_of_a_product_with_parts():
    """Chunks of 128 k and a workgroup a compute unit; chunks of 64 and two a unit where a part would be longer than
    1024 k, up to 128 rows; never more than 16 parts."""
    from infinilm_amd import kernels as K
    assert K._tall_plan(64, 4096, 4096) == (128, 8, 4)       # o projection of the 8B shape: 32 tiles x 8 parts
    assert K._tall_plan(64, 4096, 16384) == (64, 16, 16)     # down projection: 32 tiles x 16 parts of 1024 k
    assert K._tall_plan(208, 4096, 16384) == (128, 8, 16)    # many rows: chunks of 128
    assert K._tall_plan(64, 2304, 5760) == (128, 15, 3)
    assert K._tall_plan(32, 128, 65536)[1] <= K.TALL_MAX_PARTS


def test_where_the_gate_up_projection_keeps_x_in_lds(K, monkeypatch):
    """17 to 112 rows, and up to 176 rows that are no multiple of 32, take the kernel with chunks of X in LDS
    when the outputs fill the chip; other row counts are left to the library's product and the activation kernel."""
    monkeypatch.setattr(K, "GATEUP_TALL_MIN_OUTPUTS", 0)
    w = _rand((2 * 96, 72), 44, torch.bfloat16, 0.1).to(DEV)
    for M, taken in ((17, True), (33, True), (65, True), (96, True), (112, True), (113, True), (128, False), (144, True), (160, False), (176, True), (192, False),
                     (175, True), (177, False), (208, False), (209, False)):
        x = _rand((M, 72), 45, torch.bfloat16).to(DEV)
        act = K.gateup_swiglu_gemm(x, w, None)
        assert (act is not None) == taken, M
        if taken:
            y = P.plain_linear(x.to(F64), w.to(F64))
            _close(act, P.plain_swiglu(y[:, :96], y[:, 96:]), 1e-2)


@pytest.mark.parametrize("M,Ko,H,I,bias,wdt", [(8, 4096, 4096, 16384, False, torch.bfloat16), (3, 96, 80, 200, True, torch.float32),
                                               (16, 1032, 328, 331, True, torch.bfloat16), (1, 2304, 2304, 5760, False, torch.float32),
                                               (20, 200, 96, 50, False, torch.float32), (32, 4096, 1024, 4096, True, torch.bfloat16),
                                               (5, 8192, 72, 61, False, torch.bfloat16)])
def test_branch_tail_and_deferred_norm(K, monkeypatch, M, Ko, H, I, bias, wdt):
    """The output projection with the residual sum and the first half of the next norm in its epilogue,
    and the gate/up projection that finishes that norm in its own: together they equal
    residual += alpha * (x Wo^T + b); swiglu(rmsnorm(residual) Wgu^T + b) of the plain formulas."""
    monkeypatch.setattr(K, "TAIL_MAX_ROWS", 32)
    x, wo = _rand((M, Ko), 51, torch.bfloat16), _rand((H, Ko), 52, torch.bfloat16, scale=2.0 * Ko ** -0.5)
    bo = _rand((H,), 53, torch.bfloat16) if bias else None
    r = _rand((M, H), 54, scale=2.0)
    nw = (_rand((H,), 55) * 0.2 + 1.0).to(wdt)
    wgu = _rand((2 * I, H), 56, torch.bfloat16, scale=2.0 * H ** -0.5)
    bgu = _rand((2 * I,), 57, torch.bfloat16) if bias else None
    dev = lambda t: None if t is None else t.to(DEV)
    alpha, eps = 0.37, 1e-5
    assert K.tail_ok(M, dev(wo), dev(bo), dev(nw), torch.bfloat16) and K.gateup_resident_ok(M, dev(wgu))
    rd = dev(r).clone()
    xw, ss = K.gemm_tail(dev(x), dev(wo), dev(bo), alpha, rd, dev(nw))
    act = K.gateup_swiglu_gemm(xw, dev(wgu), dev(bgu), row_ss=ss, eps=eps)
    r_want = r.to(F64) + P.plain_linear(x.to(F64), wo.to(F64), None if bo is None else bo.to(F64), alpha)
    _close(rd, r_want, 2e-5)
    assert rel_sum_sq(ss, rd, M) < 1e-5
    y = P.plain_linear(P.plain_rmsnorm(r_want, nw.to(F64), eps), wgu.to(F64), None if bgu is None else bgu.to(F64))
    _close(act, P.plain_swiglu(y[:, :I], y[:, I:]), 1.5e-2)
    # and against the three kernels it stands for (same places of rounding but one: r * w is rounded before the division)
    r2 = dev(r).clone()
    x2 = K.add_rmsnorm(r2, K.gemm(dev(x), dev(wo), dev(bo), 1.0, allow_parts=True), dev(nw), alpha, eps, torch.bfloat16)
    two = K.gateup_swiglu_gemm(x2, dev(wgu), dev(bgu))
    assert (act.float() - two.float()).abs().max() <= 2 ** -5 * max(float(two.float().abs().max()), 1e-6)
    _close(rd, r2, 1e-6)
    assert not K.tail_ok(33, dev(wo), dev(bo), dev(nw), torch.bfloat16)
    assert not K.tail_ok(M, dev(wo), dev(bo), dev(nw), torch.float32)


def rel_sum_sq(ss, r, M):
    """Relative error of the rows' sums of squares formed from the tiles' partial sums."""
    got = ss.to(F64).sum(0)[:M].cpu()
    want = (r.to(F64) ** 2).sum(1).cpu()
    return float(((got - want).abs() / want).max())


def _paged(k, v, page, n_pages, seed, dtype):
    """Scatters contiguous per-request keys/values [n, nkv, d] into a paged cache with a shuffled
    block table; unused slots hold large finite garbage so that a read beyond a length shows."""
    nkv, d = k[0].shape[1], k[0].shape[2]
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.full((n_pages, nkv, page, d), 7.0, dtype=dtype)
    vc = torch.full((n_pages, nkv, d, page), -9.0, dtype=dtype)
    tables = []
    for kr, vr in zip(k, v):
        n = kr.shape[0]
        tab = [perm.pop() for _ in range(-(-n // page))]
        for i in range(n):
            kc[tab[i // page], :, i % page, :] = kr[i].to(dtype)
            vc[tab[i // page], :, :, i % page] = vr[i].to(dtype)
        tables.append(tab)
    width = max(len(t) for t in tables)
    bt = torch.full((len(tables), width), -1, dtype=torch.int32)
    for i, t in enumerate(tables):
        bt[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return kc, vc, bt


def _attention_case(K, dtype, nh, nkv, d, page, lens, qlens, window=0, seed=0, spike=False, ramp=0.0):
    """Requests with `lens[i]` cached keys of which the last `qlens[i]` are this step's queries."""
    ks = [_rand((n, nkv, d), seed + 10 * i + 1, dtype) for i, n in enumerate(lens)]
    vs = [_rand((n, nkv, d), seed + 10 * i + 2, dtype) for i, n in enumerate(lens)]
    qs = [_rand((n, nh, d), seed + 10 * i + 3, dtype) for i, n in enumerate(lens)]
    if spike:
        # one far key per request must dominate: its score stands out by construction
        for q, k in zip(qs, ks):
            far = 3 if k.shape[0] > 3 else 0
            k[far] = (q[-1, 0:1, :].float() * 4.0 / math.sqrt(d)).to(dtype)
    if ramp:
        # scores of the last query's first head rise by `ramp` (natural units) a key: the running
        # maximum moves in every tile, by little or by much
        for q, k in zip(qs, ks):
            u = q[-1, 0, :].float()
            u = u / (u @ u)
            k[:, 0, :] = (k[:, 0, :].float() + torch.arange(k.shape[0])[:, None] * (ramp * math.sqrt(d)) * u).to(dtype)
    n_pages = sum(-(-n // page) for n in lens) + 3
    kc, vc, bt = _paged(ks, vs, page, n_pages, seed, dtype)
    q_rows, seg, pos = [], [], []
    for i, (n, ql) in enumerate(zip(lens, qlens)):
        q_rows.append(qs[i][n - ql:])
        seg += [i] * ql
        pos += list(range(n - ql, n))
    q = torch.cat(q_rows).reshape(-1, nh * d)
    # work lists as the step function builds them: runs of up to 8 tokens of a request, and single tokens
    tiles, singles, row = [], [], 0
    for ql in qlens:
        if ql == 1:
            singles.append(row)
        else:
            for k in range(0, ql, 8):
                tiles += [row + k, min(8, ql - k)]
        row += ql
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    extra = dict(tiles=i32(tiles).view(-1, 2), single_rows=i32(singles) if singles else None) if tiles else {}
    out = K.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), torch.tensor(seg, dtype=torch.int32, device=DEV),
                            torch.tensor(pos, dtype=torch.int32, device=DEV), nh, nkv, d, 1 / math.sqrt(d), window,
                            max_total_len=max(lens), **extra)
    want = []
    for i, (n, ql) in enumerate(zip(lens, qlens)):
        last = P.plain_attention(qs[i].to(F64), ks[i].to(F64), vs[i].to(F64), 1 / math.sqrt(d), window, first_row=n - ql)
        want.append(last.reshape(ql, nh * d))
    return out, torch.cat(want)


@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (3, 1, 32, 8), (6, 3, 48, 16), (5, 5, 80, 7), (2, 1, 256, 16),
                                           (32, 2, 128, 64), (34, 2, 64, 12), (5, 1, 40, 8), (3, 3, 112, 20)])
def test_attention_float32(K, nh, nkv, d, page):
    """Heads in steps of 16 over pages that are multiples of 4 take the float matrix-core kernel (groups of up to
    16 heads side by side, groups of 17 in two parts); other head and page sizes the plain kernel."""
    out, want = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[1, 70, 33, 130], qlens=[1, 70, 1, 5])
    _close(out, want, 3e-6)
    out, want = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[90, 20], qlens=[2, 20], window=11, seed=5)
    _close(out, want, 3e-6)
    out, want = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[300, 65], qlens=[1, 1], seed=9, spike=True)
    _close(out, want, 3e-6)


def test_attention_float32_one_wave_a_chunk_gives_the_same_bits(K, monkeypatch):
    """The plain kernel's two launch shapes (one wave walks all chunks of a token and head; one wave a
    chunk and a fold) agree bit for bit, so that a token decoded alone and the same token inside a
    portion of a prompt cannot differ."""
    case = dict(lens=[1500, 700, 513, 40], qlens=[1, 1, 3, 1])
    for window in (0, 600):
        monkeypatch.setattr(K, "BASIC_SPLIT", True)
        split, want = _attention_case(K, torch.float32, 6, 2, 48, 7, window=window, seed=4, **case)
        monkeypatch.setattr(K, "BASIC_SPLIT", False)
        whole, _ = _attention_case(K, torch.float32, 6, 2, 48, 7, window=window, seed=4, **case)
        assert torch.equal(split.cpu(), whole.cpu())
        _close(split, want, 3e-6)


@pytest.mark.parametrize("nh,nkv,d,page", [(6, 2, 48, 8), (32, 2, 128, 64), (17, 1, 32, 4)])
def test_attention_float32_matrix_cores_one_wave_a_chunk_gives_the_same_bits(K, monkeypatch, nh, nkv, d, page):
    """The float matrix-core kernel's two launch shapes agree bit for bit, with and without a window whose
    edge falls inside a chunk, and a token gives the same bits alone as inside a batch of portions."""
    case = dict(lens=[1500, 700, 513, 40], qlens=[1, 1, 3, 1])
    for window in (0, 600, 100):
        monkeypatch.setattr(K, "F32_ATTN_SPLIT", True)
        split, want = _attention_case(K, torch.float32, nh, nkv, d, page, window=window, seed=4, **case)
        monkeypatch.setattr(K, "F32_ATTN_SPLIT", False)
        whole, _ = _attention_case(K, torch.float32, nh, nkv, d, page, window=window, seed=4, **case)
        assert torch.equal(split.cpu(), whole.cpu())
        _close(split, want, 3e-6)
    monkeypatch.setattr(K, "F32_ATTN_SPLIT", True)
    alone, _ = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[1500], qlens=[1], seed=4)
    among, _ = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[1500, 700, 513], qlens=[40, 700, 2], seed=4)
    assert torch.equal(alone.cpu()[0], among.cpu()[39])


def test_attention_float32_refuses_a_bound_below_a_position_loudly(K):
    """A caller's bound on the lengths that is too small for a token must not lose a chunk silently: the
    fold marks the token's row with NaNs."""
    nh, nkv, d, page = 4, 2, 32, 16
    out, want = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[700, 300], qlens=[1, 1], seed=2)
    _close(out, want, 3e-6)
    import infinilm_amd.kernels as kk
    orig = kk.paged_attention
    try:
        kk.paged_attention = lambda *a, **kw: orig(*a, **dict(kw, max_total_len=400))
        bad, _ = _attention_case(K, torch.float32, nh, nkv, d, page, lens=[700, 300], qlens=[1, 1], seed=2)
    finally:
        kk.paged_attention = orig
    assert torch.isnan(bad[0]).all() and not torch.isnan(bad[1]).any()


@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 16), (3, 1, 32, 16), (6, 3, 48, 32), (32, 2, 128, 64), (16, 16, 64, 16),
                                            (34, 2, 80, 16), (5, 1, 112, 48)])
def test_attention_bfloat16_matrix_cores(K, nh, nkv, d, page):
    # whole prompts, decode rows, a portion with history, lengths that cross key chunks of 256
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[1, 70, 33, 300], qlens=[1, 70, 1, 9])
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[700, 257, 256, 31], qlens=[1, 1, 1, 31], seed=3)
    _close(out, want, 1.2e-2)
    # a window's edge, inside a page and across chunks
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[90, 20, 600], qlens=[2, 20, 3], window=11, seed=5)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[600, 40], qlens=[1, 40], window=300, seed=6)
    _close(out, want, 1.2e-2)
    # a far key among hundreds must dominate
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[520, 65], qlens=[1, 1], seed=9, spike=True)
    _close(out, want, 1.2e-2)


@pytest.mark.parametrize("ramp", [0.02, 0.7, -0.05])
def test_attention_bfloat16_with_a_moving_maximum(K, ramp):
    """The tile kernel moves its exponent's reference point lazily: rising and falling scores."""
    out, want = _attention_case(K, torch.bfloat16, 32, 2, 128, 64, lens=[700, 130], qlens=[300, 130], seed=11, ramp=ramp)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, 6, 3, 48, 16, lens=[500, 9], qlens=[77, 9], seed=12, ramp=ramp, window=200)
    _close(out, want, 1.2e-2)


@pytest.mark.parametrize("d,page,window", [(128, 64, 128), (128, 64, 256), (64, 128, 192), (32, 256, 64)])
def test_attention_bfloat16_window_edge_on_a_tile_boundary(K, d, page, window):
    """A long portion under a window that is a multiple of the 64-key tile: one tile of tokens in
    eight has its last token's window begin exactly where a key tile begins, so that token sees
    nothing of the tile before (all its scores there are masked while it has seen no key yet) and
    the next tile takes the mask-free path."""
    out, want = _attention_case(K, torch.bfloat16, 4, 2, d, page, lens=[704, 333], qlens=[256, 200], window=window, seed=21)
    _close(out, want, 1.2e-2)


@pytest.mark.parametrize("nh,nkv,d,page", [(32, 2, 128, 256), (4, 2, 64, 128), (6, 3, 48, 256), (3, 1, 32, 128)])
def test_attention_bfloat16_pages_longer_than_a_key_tile(K, nh, nkv, d, page):
    """Pages of 128 and 256 keys: a 64-key tile begins in the middle of a page; portions with
    history, decoded tokens beside them, a far key that dominates."""
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[700, 300, 65, 1], qlens=[100, 1, 65, 1], seed=31)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[520, 900], qlens=[9, 1], seed=32, spike=True)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[600, 258], qlens=[77, 2], seed=33, window=130)
    _close(out, want, 1.2e-2)


@pytest.mark.parametrize("nh,nkv,d,page,lens", [(4, 2, 64, 64, [20000, 9000]), (8, 2, 128, 256, [16500]), (3, 1, 48, 16, [5000, 3300, 70])])
def test_attention_bfloat16_few_tokens_over_many_chunks(K, nh, nkv, d, page, lens):
    """One or two decoded tokens over tens of thousands of keys: up to 256 chunks, merged by the kernel of
    four waves (a quarter of the chunks each) instead of the one of one wave; a far key that dominates, a
    window that leaves most chunks out."""
    span, nsplit = K.attention_chunks(max(lens), page, K.bound_rows(len(lens)) * nkv, torch.device(DEV))
    assert nsplit > 24 and nsplit <= K.ATT_MAX_CHUNKS   # the merge of four waves
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=lens, qlens=[1] * len(lens), seed=41)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=lens, qlens=[1] * len(lens), seed=42, spike=True)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=lens, qlens=[1] * len(lens), seed=43, window=max(lens) // 2 + 77)
    _close(out, want, 1.2e-2)


@pytest.mark.parametrize("nh,nkv,d,page,n", [(8, 8, 64, 16, 40), (32, 2, 128, 64, 150), (4, 1, 32, 16, 120)])
def test_attention_bfloat16_many_single_tokens(K, nh, nkv, d, page, n):
    """Many decoded tokens in one launch: the chunks get long (several 128-key steps a workgroup,
    loads a step ahead), contexts from one key to a thousand."""
    g = torch.Generator().manual_seed(n)
    lens = torch.randint(1, 1000, (n,), generator=g).tolist()
    lens[0], lens[1], lens[2] = 1, 1000, 129
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=lens, qlens=[1] * n, seed=n)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=lens, qlens=[1] * n, seed=n + 1, window=200)
    _close(out, want, 1.2e-2)


def test_attention_bfloat16_with_a_block_table_beyond_lds(K):
    """33,000 keys in pages of 16: more block-table entries than the tile kernel keeps in LDS, and
    the most chunks the single-token kernel cuts a context into."""
    out, want = _attention_case(K, torch.bfloat16, 4, 2, 64, 16, lens=[33000, 50], qlens=[11, 1], seed=41)
    _close(out, want, 1.2e-2)
    out, want = _attention_case(K, torch.bfloat16, 4, 2, 64, 16, lens=[33000, 70], qlens=[1, 1], seed=42)
    _close(out, want, 1.2e-2)


def test_attention_does_not_depend_on_the_batch(K):
    """The same token alone and inside a larger batch gives the same bits (bfloat16 kernel), as long
    as both launches cut the context into chunks of the same length (few tokens: always 128 keys)."""
    nh, nkv, d, page = 8, 2, 64, 16
    out_a, _ = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[300], qlens=[1], seed=0)
    out_b, _ = _attention_case(K, torch.bfloat16, nh, nkv, d, page, lens=[300, 50, 700], qlens=[1, 50, 2], seed=0)
    assert torch.equal(out_a.cpu()[0], out_b.cpu()[0])


def test_argmax_and_sampling(K):
    V = 73448
    logits = _rand((5, V), 20, scale=3.0)
    logits[1, 100] = logits[1, 70000] = 50.0      # a tie: the first index wins
    logits[2, V - 1] = 60.0
    dl = logits.to(DEV)
    assert K.argmax(dl).tolist() == [int(torch.argmax(logits[0])), 100, V - 1, int(torch.argmax(logits[3])), int(torch.argmax(logits[4]))]

    def run(temp, k, p, u, rows=logits):
        n = rows.shape[0]
        mk = lambda v, dt: torch.tensor([v] * n if not isinstance(v, list) else v, dtype=dt, device=DEV)
        return K.sample(rows.to(DEV), mk(temp, torch.float32), mk(k, torch.int32), mk(p, torch.float32),
                        mk(u, torch.float32)).tolist()

    assert run(1.0, 1, 1.0, 0.5) == K.argmax(dl).tolist()           # top_k 1 is greedy
    # a greedy row beside sampled rows, index 0 tied for the maximum: the first index wins there too
    tie = logits.clone()
    tie[0, 0] = tie[0, 5000] = tie[3, 0] = tie[3, V - 1] = 70.0
    mixed = run([0.0, 1.0, 0.8, 1.0, 0.0], [0, 1, 40, 1, 0], 1.0, 0.3, tie)
    assert mixed[0] == 0 and mixed[3] == 0 and mixed[1] == 100 and mixed[4] == int(torch.argmax(logits[4]))
    assert run(0.0, 0, 1.0, 0.9) == K.argmax(dl).tolist()           # temperature 0 is greedy
    # inverse CDF in vocabulary order against the plain implementation, over many u
    small = _rand((1, 331), 21, scale=2.0)
    for temp, k, p in [(0.8, 0, 1.0), (1.3, 5, 1.0), (1.0, 0, 0.6), (0.7, 40, 0.9), (1.0, 331, 1.0), (2.0, 2, 0.5)]:
        dist = P.plain_sample_distribution(small[0], temp, k, p)
        cdf = torch.cumsum(dist, 0)
        us = [i / 64.0 + 1 / 128.0 for i in range(64)]
        got = run(temp, k, p, us, small.expand(64, 331).contiguous())
        for u, tok in zip(us, got):
            assert dist[tok] > 0, f"token {tok} is outside the kept set (T={temp}, k={k}, p={p})"
            lo = float(cdf[tok] - dist[tok])
            assert lo - 1e-4 <= u <= float(cdf[tok]) + 1e-4, f"u={u} not in token {tok}'s interval"
    # every row length takes its own kernel shape (row in registers of 1024 or 512 threads, or streamed)
    for Vn in (16384, 20000, 40000, 73448, 90000, 122753):
        big = _rand((1, Vn), 30 + Vn % 7, scale=2.5)
        for temp, k, p in [(0.9, 0, 1.0), (1.1, 50, 0.9), (1.0, 0, 0.7), (0.6, 7, 1.0)]:
            dist = P.plain_sample_distribution(big[0], temp, k, p)
            cdf = torch.cumsum(dist, 0)
            us = [i / 8.0 + 1 / 16.0 for i in range(8)]
            got = run(temp, k, p, us, big.expand(8, Vn).contiguous())
            for u, tok in zip(us, got):
                assert dist[tok] > 0, f"V={Vn}: token {tok} is outside the kept set (T={temp}, k={k}, p={p})"
                lo = float(cdf[tok] - dist[tok])
                assert lo - 2e-4 <= u <= float(cdf[tok]) + 2e-4, f"V={Vn}: u={u} not in token {tok}'s interval"
    # frequencies over many draws follow the probabilities
    dist = P.plain_sample_distribution(small[0], 1.0, 8, 1.0)
    n = 4096
    g = torch.Generator().manual_seed(1)
    us = torch.rand(n, generator=g).tolist()
    got = torch.tensor(run(1.0, 8, 1.0, us, small.expand(n, 331).contiguous()))
    freq = torch.bincount(got, minlength=331).to(F64) / n
    assert float((freq - dist).abs().max()) < 0.03
    # the big vocabulary: top-k keeps exactly the k largest
    top = set(torch.topk(logits[0], 3).indices.tolist())
    for u in (0.01, 0.4, 0.99):
        assert run(1.5, 3, 1.0, u, logits[:1])[0] in top
