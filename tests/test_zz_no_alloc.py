"""The attention entry point that allocates nothing (`ilm_attn_mfma_static`, csrc/no_alloc.h), called
through ctypes as a caller without an allocator would, against `ilm_attn_mfma` with a workspace
the caller brings: two calls in a row on the same GPU, the second with a smaller input (the
scratch keeps the first call's contents), and a size beyond the scratch, which must be refused."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(seed, lens, nh, nkv, d, page):
    """Random queries, a paged cache with a shuffled block table and the metadata of one decoded
    token a request."""
    g = torch.Generator().manual_seed(seed)
    n = len(lens)
    pages_of = [-(-l // page) for l in lens]
    n_pages = sum(pages_of) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    bt = torch.full((n, max(pages_of)), -1, dtype=torch.int32)
    for i, k in enumerate(pages_of):
        bt[i, :k] = torch.tensor([perm.pop() for _ in range(k)], dtype=torch.int32)
    dev = lambda t: t.to(DEV)
    return {
        "q": dev(torch.randn((n, nh * d), generator=g).to(torch.bfloat16)),
        "kc": dev(torch.randn((n_pages, nkv, page, d), generator=g).to(torch.bfloat16)),
        "vc": dev(torch.randn((n_pages, nkv, d, page), generator=g).to(torch.bfloat16)),
        "bt": dev(bt), "seg": dev(torch.arange(n, dtype=torch.int32)),
        "pos": dev(torch.tensor([l - 1 for l in lens], dtype=torch.int32)),
        "n": n, "nh": nh, "nkv": nkv, "d": d, "page": page, "width": bt.shape[1], "longest": max(lens),
    }


def _plain(c):
    """softmax(q k^T / sqrt(d)) v over each request's own keys in float64, gathered through the block table."""
    n, nh, nkv, d, page = c["n"], c["nh"], c["nkv"], c["d"], c["page"]
    out = torch.zeros((n, nh, d), dtype=torch.float64)
    q = c["q"].cpu().double().view(n, nh, d)
    kc, vc, bt, pos = c["kc"].cpu().double(), c["vc"].cpu().double(), c["bt"].cpu(), c["pos"].cpu()
    for i in range(n):
        L = int(pos[i]) + 1
        pages = bt[i, :-(-L // page)].long()
        k = kc[pages].permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :L]                  # [nkv, L, d]
        v = vc[pages].permute(1, 2, 0, 3).reshape(nkv, d, -1)[:, :, :L]               # [nkv, d, L]
        for h in range(nh):
            g = h // (nh // nkv)
            p = torch.softmax(k[g] @ q[i, h] / math.sqrt(d), 0)
            out[i, h] = v[g] @ p
    return out.view(n, nh * d)


def _launch_static(L, c, span, out):
    """The call itself, on the current stream, without waiting (so that it can be recorded)."""
    n, nh, d = c["n"], c["nh"], c["d"]
    nsplit = -(-c["longest"] // span)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    return L.ilm_attn_mfma_static(ptr(out), ptr(c["q"]), ptr(c["kc"]), ptr(c["vc"]), ptr(c["bt"]), ptr(c["seg"]), ptr(c["pos"]),
                                  None, n, nh, c["nkv"], d, c["page"], c["width"], nh * d, nh * d, 1.0 / math.sqrt(d), 0,
                                  nsplit, span, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))


def _run(L, c, span, static):
    n, nh, d = c["n"], c["nh"], c["d"]
    nsplit = -(-(int(c["pos"].max()) + 1) // span)
    out = torch.full((n, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tail = (n, nh, c["nkv"], d, c["page"], c["width"], nh * d, nh * d, 1.0 / math.sqrt(d), 0, nsplit, span, stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    common = (ptr(c["q"]), ptr(c["kc"]), ptr(c["vc"]), ptr(c["bt"]), ptr(c["seg"]), ptr(c["pos"]), None)
    if static:
        rc = L.ilm_attn_mfma_static(ptr(out), *common, *tail)
    else:
        ws_acc = torch.empty((n * nh * nsplit * d,), dtype=torch.float32, device=DEV)
        ws_ml = torch.empty((n * nh * nsplit * 2,), dtype=torch.float32, device=DEV)
        rc = L.ilm_attn_mfma(ptr(out), ptr(ws_acc), ptr(ws_ml), *common, *tail)
    torch.cuda.synchronize()
    return rc, out


def test_attention_without_allocation_equals_the_one_with_a_workspace():
    from infinilm_amd.csrc import lib

    L = lib.load()
    assert L.ilm_attn_static_scratch_floats() == 4 << 20
    big = _case(1, [1000, 129, 517, 2048, 1, 300, 777, 1500], nh=32, nkv=2, d=128, page=64)
    small = _case(2, [260, 40, 131], nh=6, nkv=3, d=48, page=16)
    for c, span in ((big, 256), (small, 128), (big, 128)):   # a large call, a smaller one, the large one again
        rc_w, want = _run(L, c, span, static=False)
        rc_s, got = _run(L, c, span, static=True)
        assert rc_w == 0 and rc_s == 0, lib.last_error()
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want), "the static-scratch call differs from the call with a workspace"
        err = float((got.cpu().double() - _plain(c)).abs().max())
        assert err < 2e-2, f"the static-scratch call against the plain formula in float64: {err:.3e}"
    # beyond the scratch: refused with a message, nothing launched
    n, nh, d = 64, 32, 128
    nsplit = (4 << 20) // (n * nh * (d + 2)) + 1
    out = torch.zeros((n, nh * d), dtype=torch.bfloat16, device=DEV)
    p = ctypes.c_void_p(out.data_ptr())
    rc = L.ilm_attn_mfma_static(p, p, p, p, p, p, p, None, n, nh, 2, d, 64, 4, nh * d, nh * d, 0.1, 0, nsplit, 128,
                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -1 and "exceed the static scratch" in lib.last_error()
    torch.cuda.synchronize()
    assert not out.any()


def test_attention_without_allocation_inside_a_recorded_graph():
    """The callers it is for: the call is recorded into a HIP graph (after ilm_attn_static_init(), so that the
    address look-up lies outside the capture) and replayed several times with new queries and eager work of the
    same entry point between the replays; every replay equals the eager call on the same inputs."""
    from infinilm_amd.csrc import lib

    L = lib.load()
    assert L.ilm_attn_static_init() == 0, lib.last_error()
    c = _case(3, [900, 64, 333, 1200], nh=32, nkv=2, d=128, page=64)
    other = _case(4, [500, 31], nh=8, nkv=2, d=64, page=16)
    out = torch.zeros((c["n"], c["nh"] * c["d"]), dtype=torch.bfloat16, device=DEV)
    assert _launch_static(L, c, 256, out) == 0, lib.last_error()     # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = _launch_static(L, c, 256, out)
    assert rc == 0, lib.last_error()
    g = torch.Generator().manual_seed(9)
    for replay in range(4):
        c["q"].copy_(torch.randn(c["q"].shape, generator=g).to(torch.bfloat16))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        # eager work on the same scratch between the replays
        rc_o, _ = _run(L, other, 128, static=True)
        rc_e, want = _run(L, c, 256, static=False)
        assert rc_o == 0 and rc_e == 0, lib.last_error()
        assert torch.equal(got, want), f"replay {replay} differs from the eager call"
    err = float((got.cpu().double() - _plain(c)).abs().max())
    assert err < 2e-2, f"replayed call against the plain formula in float64: {err:.3e}"
