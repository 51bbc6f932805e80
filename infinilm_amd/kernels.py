"""Typed Python faces of the HIP kernels.

Each function checks what the kernel assumes about its operands (device, dtype, contiguity,
shapes) on the host before the launch, and raises `KernelError` with the kernel's own message
when it refuses a size.  Nothing here computes on the CPU or through a tensor library: a missing
library or a CPU tensor is an error.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from .csrc import lib as _libmod

F32 = torch.float32
BF16 = torch.bfloat16
_DT = {torch.float32: 0, torch.bfloat16: 1}
ATT_TILE_TOKENS = 8  # tokens per tile of the prompt-portion attention kernel (ilm_attn_tile_tokens())
ATT_STEP = 128  # keys a workgroup of the chunked attention takes in one step (ilm_attn_mfma_step())
ATT_MAX_CHUNKS = 256  # most chunks a context is cut into (a wave of the merge kernel walks a quarter of them; it takes 512)
BASIC_CHUNK = 512    # keys a chunk of the plain attention kernel (ilm_attn_basic_chunk())
BASIC_SPLIT = os.environ.get("INFINILM_AMD_BASIC_SPLIT", "1") == "1"   # 0: always one wave a (token, head)
BASIC_SPLIT_WAVES = 4096   # (token, head) pairs up to which the plain kernel takes one wave a chunk
F32_ATTN_CHUNK = 128   # keys a chunk of the 32-bit matrix-core attention (ilm_attn_f32_chunk())
F32_ATTN_SPLIT = os.environ.get("INFINILM_AMD_F32_ATTN_SPLIT", "1") == "1"   # 0: always one wave a (token, head group)
F32_ATTN_SPLIT_WAVES = 2048   # (token, head group) pairs up to which it takes one wave a chunk
# INFINILM_AMD_BASIC=1 runs the plain kernels everywhere (for telling a kernel's fault from the engine's)
FORCE_BASIC = os.environ.get("INFINILM_AMD_BASIC", "0") == "1"
SKINNY_VARIANT = int(os.environ.get("INFINILM_AMD_SKINNY_VARIANT", "0"))  # 0: the kernel chooses
USE_KSPLIT = os.environ.get("INFINILM_AMD_KSPLIT", "1") == "1"
USE_LIBRARY_GEMM = os.environ.get("INFINILM_AMD_LIBRARY_GEMM", "1") == "1"


class KernelError(RuntimeError):
    pass


def _lib():
    return _libmod.load()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (the raw lookup costs a tenth of `torch.cuda.current_stream()`,
    which matters with some hundred launches a step)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


# ---- timers per kernel entry point, off unless asked for ------------------------------------------
_TIMES: Optional[dict] = {} if os.environ.get("INFINILM_AMD_KERNEL_TIMES", "0") == "1" else None


def enable_timing(on: bool = True) -> None:
    """Brackets every launch with a pair of events (also: INFINILM_AMD_KERNEL_TIMES=1).  Launches
    inside a graph capture are not timed.  Costs host time; for looking at a step, not for serving."""
    global _TIMES
    _TIMES = {} if on else None


def timing_report(reset: bool = True) -> dict:
    """{entry point: {"calls", "total_ms", "mean_us"}}, after waiting for the device."""
    if _TIMES is None:
        return {}
    torch.cuda.synchronize()
    out = {}
    for name, pairs in _TIMES.items():
        total = sum(a.elapsed_time(b) for a, b in pairs)
        out[name] = {"calls": len(pairs), "total_ms": round(total, 4), "mean_us": round(1e3 * total / max(len(pairs), 1), 2)}
    if reset:
        _TIMES.clear()
    return dict(sorted(out.items(), key=lambda kv: -kv[1]["total_ms"]))


class _timed:
    """Context of one launch; a no-op when timing is off or the stream is being captured."""
    __slots__ = ("name", "start")

    def __init__(self, name: str):
        self.name = name
        self.start = None

    def __enter__(self):
        if _TIMES is not None and not torch.cuda.is_current_stream_capturing():
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if self.start is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _TIMES.setdefault(self.name, []).append((self.start, end))
        return False


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; the kernels take float32 and bfloat16") from None


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelError("the kernels run on the GPU only; got a CPU tensor")


def _run(name: str, *args) -> None:
    if _TIMES is None:
        rc = getattr(_lib(), name)(*args)
    else:
        with _timed(name):
            rc = getattr(_lib(), name)(*args)
    if rc != 0:
        raise KernelError(_libmod.last_error())


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, nkv: int, d: int) -> int:
    """Keys [pages, nkv, page, d], values transposed [pages, nkv, d, page]; returns the page size."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != d \
            or tuple(v_cache.shape) != (k_cache.shape[0], nkv, d, k_cache.shape[2]) \
            or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError(f"cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} are not "
                          f"[pages, {nkv}, page, {d}] / [pages, {nkv}, {d}, page]")
    return k_cache.shape[2]


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor, got {t.dtype}")


# ------------------------------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """float32 residual rows scale * table[ids]."""
    _dev(ids, table)
    _i32(ids, "ids")
    V, H = table.shape
    if not table.is_contiguous():
        raise KernelError("embedding table must be contiguous")
    T = ids.numel()
    out = torch.empty((T, H), dtype=F32, device=table.device)
    _run("ilm_embed", out.data_ptr(), ids.data_ptr(), table.data_ptr(), T, H, V, float(scale), _dt(table), _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, branch: Optional[torch.Tensor], weight: torch.Tensor,
                alpha: float, eps: float, out_dtype: torch.dtype, frag: bool = False):
    """residual += alpha * branch (in place, float32), then its RMS norm times weight, as out_dtype.
    `frag`: the result comes in fragment order (`FragRows`; bfloat16, at most 64 rows of a multiple of 8 elements),
    for a product that takes it so.

    `branch` is [rows, H] in out_dtype or float32, or [parts, rows, H] (the float32 parts of a K-split
    product, summed in order)."""
    _dev(residual, branch, weight)
    rows, H = residual.shape
    if residual.dtype != F32 or not residual.is_contiguous():
        raise KernelError("the residual stream is a contiguous float32 tensor")
    parts, pstride, h_dt = 1, 0, _DT[out_dtype]
    if branch is not None:
        if branch.dim() == 3:
            parts, pstride = branch.shape[0], branch.stride(0)
        if tuple(branch.shape[-2:]) != (rows, H) or branch.dtype not in (out_dtype, F32) or not branch.is_contiguous():
            raise KernelError(f"branch {tuple(branch.shape)} {branch.dtype} does not match residual "
                              f"{tuple(residual.shape)} / {out_dtype}")
        h_dt = _dt(branch)
    if weight.shape != (H,) or not weight.is_contiguous():
        raise KernelError(f"norm weight has shape {tuple(weight.shape)}, expected ({H},)")
    if frag:
        if out_dtype != BF16 or rows > FRAG_MAX_ROWS or H % 8:
            raise KernelError("a norm's result in fragment order is bfloat16, at most 64 rows of a multiple of 8 elements")
        out = frag_rows_empty(rows, H, residual.device)
        _run("ilm_add_rmsnorm", out.data.data_ptr(), residual.data_ptr(), _ptr(branch), weight.data_ptr(), rows, H,
             float(alpha), float(eps), _DT[out_dtype], _dt(weight), h_dt, parts, pstride, -(-rows // 16), _stream())
        return out
    out = torch.empty((rows, H), dtype=out_dtype, device=residual.device)
    _run("ilm_add_rmsnorm", out.data_ptr(), residual.data_ptr(), _ptr(branch), weight.data_ptr(), rows, H,
         float(alpha), float(eps), _DT[out_dtype], _dt(weight), h_dt, parts, pstride, 0, _stream())
    return out


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                 k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                 slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, rd: int) -> None:
    """Rotates q and k inside the fused projection rows [T, (nh + 2 nkv) d] and writes k, v to the
    paged cache [pages, nkv, page, d] at `slots` (None: no write)."""
    _dev(qkv, positions, cos, sin, k_cache, v_cache, slots)
    _i32(positions, "positions")
    T = qkv.shape[0]
    if qkv.stride(1) != 1 or positions.numel() != T:
        raise KernelError("qkv rows must be dense and positions must have one entry a token")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or (rd > 0 and cos.shape[1] != rd // 2):
        raise KernelError(f"rotation tables must be float32 [positions, {rd // 2}], got {tuple(cos.shape)}")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    _run("ilm_rope_kvwrite", qkv.data_ptr(), positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache),
         _ptr(v_cache), _ptr(slots), T, nh, nkv, d, rd, qkv.stride(0), page, _dt(qkv), _stream())


USE_QKV_ROPE = os.environ.get("INFINILM_AMD_QKV_ROPE", "1") == "1"


def qkv_rope_gemm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                  cos: torch.Tensor, sin: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], nh: int, nkv: int, d: int, rd: int) -> Optional[torch.Tensor]:
    """The fused projection x w^T (+ bias) of a few rows, q and k rotated and k, v written to the cache
    in the product's epilogue.  Returns the rotated q [T, nh*d], or None where the fused kernel does
    not apply (more than 32 rows, float32, a partly rotated or odd-sized head): the caller then
    runs the projection and `rope_kvwrite` one after the other."""
    M, K = x.shape
    if not (USE_QKV_ROPE and not FORCE_BASIC and x.dtype == BF16 and w.dtype == BF16 and _few_rows(M, K) and rd == d and d % 32 == 0
            and K % 8 == 0 and K <= 8192 and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return None
    _dev(x, w, bias, positions, cos, sin, k_cache, v_cache, slots)
    _i32(positions, "positions")
    if w.shape != ((nh + 2 * nkv) * d, K) or positions.numel() != M:
        raise KernelError(f"fused projection {tuple(w.shape)} does not fit {nh}+2*{nkv} heads of {d} over {K}")
    if bias is not None and (bias.shape != (w.shape[0],) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused projection")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or cos.shape[1] != d // 2 \
            or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError(f"rotation tables must be float32 [positions, {d // 2}], got {tuple(cos.shape)}")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != BF16 or v_cache.dtype != BF16:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    q = torch.empty((M, nh * d), dtype=BF16, device=x.device)
    _run("ilm_gemm_qkv_rope", q.data_ptr(), q.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), _ptr(bias),
         M, K, positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache) if slots is not None else None,
         _ptr(v_cache) if slots is not None else None, _ptr(slots), nh, nkv, d, page, _stream())
    return q


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up from rows [gate | up]."""
    _dev(gate_up)
    T, two_i = gate_up.shape
    if two_i % 2 or gate_up.stride(1) != 1:
        raise KernelError("swiglu takes dense rows of even length")
    out = torch.empty((T, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _run("ilm_swiglu", out.data_ptr(), gate_up.data_ptr(), T, two_i // 2, gate_up.stride(0), _dt(gate_up), _stream())
    return out


def gather_rows(x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    _dev(x, idx)
    _i32(idx, "row indices")
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("gather_rows takes a contiguous matrix")
    out = torch.empty((idx.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    _run("ilm_gather_rows", out.data_ptr(), x.data_ptr(), idx.data_ptr(), idx.numel(), x.shape[1], _dt(x), _stream())
    return out


_LIBRARY_F32_OUT = [True]   # cleared when torch.mm refuses out_dtype
KSPLIT_SPAN = 4096  # K range of one part of the K-split few-rows product (ilm_gemm_ksplit_max_k(1))
# Rows up to which the products keep X in registers (16 or 32; 32 only for K up to 4096 a workgroup)
FEW_ROWS = int(os.environ.get("INFINILM_AMD_FEW_ROWS", "32"))


def _few_rows(M: int, K: int) -> bool:
    """Whether the products that keep X in registers take M rows: a wave of eight holds the fragments of K / 8 of one
    group of 16 rows in 4 registers a 32 k, and 256 registers take 16 rows of K up to 8192 or 32 rows of K up to 4096
    beside the W fragments in flight."""
    groups = max(1, min(FEW_ROWS // 16, 8192 // max(K, 4096)))
    return M <= 16 * groups


def _frag_of(frag_w):
    """`frag_w` arguments are a FragWeight, a function that packs one when it is needed, or None."""
    return frag_w() if callable(frag_w) else frag_w


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, alpha: float = 1.0,
         out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
         allow_parts: bool = False, frag_w=None) -> torch.Tensor:
    """alpha * (a w^T + bias); a [M, K] with dense rows, w [N, K]; float accumulation.

    `allow_parts`: the result goes straight into the residual sum (add_rmsnorm), so it may come in
    float32 instead of the activations' dtype, and in parts [P, M, N] that still have to be summed;
    parts are chosen for few rows and long K, where splitting K over workgroups pays."""
    _dev(a, w, bias, out)
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelError(f"gemm shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
    if a.dtype != w.dtype or a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm operands must share a dtype and have dense rows")
    M, K = a.shape
    N = w.shape[0]
    out_dtype = out_dtype or a.dtype
    if bias is not None and (bias.shape != (N,) or bias.dtype != w.dtype or not bias.is_contiguous()):
        raise KernelError(f"bias shape {tuple(bias.shape)} does not fit {N} outputs")
    if out is not None and (out.shape != (M, N) or out.dtype != out_dtype or out.stride(1) != 1):
        raise KernelError("gemm output does not fit")
    fast = a.dtype == BF16 and not FORCE_BASIC
    aligned = K % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 \
        and w.data_ptr() % 16 == 0
    plain = bias is None and alpha == 1.0
    # (From 65 rows on the vendor library leaves the chip idle on such products: down projection 68 us at 96 rows, 81
    # at 128, 92 at 160, 114 at 192, 63 at 208; o projection 22, 25, 32 at 192.  Not for small matrices, whose few
    # tiles leave most of the chip idle whatever the split: 0.5B shape at 128 rows 2.22 against 1.96 ms a step with
    # the library.)
    # 17 to 208 rows on their way into the residual sum: chunks of X resident in LDS, two workgroups a compute unit
    # (gemm_tall.hip).  Measured at the 8B shapes against the kernels it took over from: o projection 9.8 us against
    # 10.6 (K ranges of 1024, X in registers) at 32 rows, 11.0 / 12.4 at 64, 12.8 / 17.1 (steps of 64 k, X through LDS, a
    # step's loads waited for before the next step's were issued) at 96, 15.8 / 19.4 at 128, 16.9 / 22.2 at 160; down projection 27.7 / 33.1 (four parts of 4096, X in registers) at
    # 32 rows, 30.3 / 33.3 at 64, 33.7 / 38.1 at 96, 37.1 / 42.0 at 128, 46.2 / 47.1 at 160, 52.0 / 56.7 at 208
    if (fast and aligned and plain and allow_parts and out is None and USE_TALL and TALL_MIN_ROWS <= M <= TALL_MAX_ROWS
            and M > 16 and _tall_fills_the_chip(N, K, a.device)):
        return _gemm_tall(a, w, K, frag_w)
    # 17 to 64 rows on their way into the residual sum: K in ranges of 1024 with the X fragments of all rows
    # in registers (o projection at 64 rows 13.1 against the library's 18.9 us, down projection 33.9
    # against 41.3, of which the sum of its 16 parts takes 5 back; up to 32 rows the down projection
    # stays with the K-split kernel and its 4 parts)
    if (fast and aligned and plain and allow_parts and out is None and 16 < M <= 64
            and -(-K // ROWS64_SPAN) <= ROWS64_MAX_PARTS and (M > FEW_ROWS or K <= KSPLIT_SPAN)):
        kb = -(-K // ROWS64_SPAN)
        parts = torch.empty((kb, M, N), dtype=F32, device=a.device)
        fw = _frag_of(frag_w) if USE_FRAG else None
        if fw is not None:   # W in fragment order: a wave's fragment is 1 KB of consecutive bytes
            _run("ilm_gemm_rows64", parts.data_ptr(), N, M * N, kb, fw.data.data_ptr(), 0, M, N, K, a.data_ptr(),
                 a.stride(0), 1, _stream())
        else:
            _run("ilm_gemm_rows64", parts.data_ptr(), N, M * N, kb, w.data_ptr(), w.stride(0), M, N, K, a.data_ptr(),
                 a.stride(0), 0, _stream())
        return parts
    if fast and aligned and plain and allow_parts and out is None and M <= max(16, FEW_ROWS) and K > KSPLIT_SPAN and USE_KSPLIT:
        kb = -(-K // KSPLIT_SPAN)
        parts = torch.empty((kb, M, N), dtype=F32, device=a.device)
        _run("ilm_gemm_ksplit", parts.data_ptr(), _DT[F32], N, M * N, kb, w.data_ptr(), w.stride(0), None, 1.0,
             M, N, K, a.data_ptr(), a.stride(0), 0, _stream())
        return parts
    few = fast and aligned and _few_rows(M, K)
    if few and allow_parts and out is None:
        out_dtype = F32   # a branch on its way into the float32 residual sum need not be rounded first
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    library_ok = fast and plain and out_dtype == BF16 and USE_LIBRARY_GEMM
    # measured at the 8B shapes: the few-rows kernel with X in registers beats the vendor library (up to
    # 32 rows: gate_up 53 against 62 us, o projection 14 against 18); where X no longer fits the
    # registers it loses (its X fragments are re-read from L2 for every 16 rows of W)
    if (not few and M > 16 and fast and bias is None and out_dtype == F32 and USE_LIBRARY_GEMM and _LIBRARY_F32_OUT[0]
            and M <= 65535):
        # bfloat16 operands, float32 accumulation and result (the output head with many rows)
        try:
            with _timed("library_gemm"):
                torch.mm(a, w.t(), out_dtype=F32, out=out)
        except (TypeError, RuntimeError) as exc:
            if "out_dtype" not in str(exc):
                raise
            _LIBRARY_F32_OUT[0] = False   # this build of the library door has no float32 result
        else:
            if alpha != 1.0:
                _run("ilm_scale_rows", out.data_ptr(), M, N, out.stride(0), float(alpha), _stream())
            return out
    if fast and aligned and M <= 64 and (few or not library_ok):
        _run("ilm_gemm_skinny", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _DT[out_dtype], SKINNY_VARIANT, _stream())
        return out
    if M > 16 and library_ok:
        # large products go to the vendor library, as the reference's linear layers do
        # (csrc/layers/quantization/none_quantization.cpp:26-46 calls its library's linear)
        with _timed("library_gemm"):
            torch.matmul(a, w.t(), out=out)
        return out
    if (a.dtype == F32 and out_dtype == F32 and not FORCE_BASIC and M <= F32_FEW_ROWS and K % 4 == 0 and a.stride(0) % 4 == 0
            and w.stride(0) % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        # the 32-bit path's few rows (decoded tokens): W streamed once on the float matrix instruction
        _run("ilm_gemm_f32_skinny", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _stream())
        return out
    if (a.dtype == F32 and out_dtype == F32 and not FORCE_BASIC and F32_FEW_ROWS > 0 and K % 4 == 0 and a.stride(0) % 4 == 0
            and w.stride(0) % 4 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        # the 32-bit path's many rows (portions of prompts): tiles on the float matrix instruction, every
        # output summed in the few-rows kernel's order, so a row's bits do not depend on the rows around it
        _run("ilm_gemm_f32_tile", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0),
             w.stride(0), out.stride(0), float(alpha), _stream())
        return out
    _run("ilm_gemm_basic", out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, a.stride(0), w.stride(0),
         out.stride(0), float(alpha), _dt(a), _DT[out_dtype], _stream())
    return out


# Rows up to which the 32-bit products take the few-rows kernel; beyond, the tile kernel that sums in the same
# order (0: neither, always the plain ascending-k kernel)
F32_FEW_ROWS = int(os.environ.get("INFINILM_AMD_F32_FEW_ROWS", "64"))


ROWS64_SPAN = 1024   # K range of one part of the 17-to-64-rows product (ilm_gemm_rows64_span())
ROWS64_MAX_PARTS = int(os.environ.get("INFINILM_AMD_ROWS64_PARTS", "16"))   # 0: never this kernel
TALL_MIN_WGS_PER_CU = 0.25   # the tall product is used where its grid can give more than a quarter of the units a workgroup


def _tall_fills_the_chip(N: int, K: int, device) -> bool:
    """The tall product cuts W into tiles of 128 rows and K into ranges of at least 512: with fewer workgroups
    than a quarter of the compute units whatever the split, the vendor library's product is faster (measured with
    the kernel this one replaced, which cut alike: the 0.5B shape's 1024 x 4096 gives 64 workgroups on 256 units and
    loses, 2.22 against 1.96 ms a step at 128 rows; the 2B-family's 2304 x 2304 gives 72 and wins)."""
    return -(-N // 128) * max(K // 512, 1) > TALL_MIN_WGS_PER_CU * _num_cus(device)


USE_TALL = os.environ.get("INFINILM_AMD_TALL", "1") == "1"
TALL_MIN_ROWS = int(os.environ.get("INFINILM_AMD_TALL_MIN_ROWS", "17"))
TALL_MAX_ROWS = 208   # most rows of X of the products that keep chunks of X in LDS (ilm_gemm_tall_max_rows())
TALL_MAX_PARTS = 16
TALL_GATEUP_MAX_ROWS = 112     # rows up to which the gate/up projection takes that product (beyond: see gateup_swiglu_gemm)


def _tall_plan(M: int, N: int, K: int) -> tuple:
    """(k a chunk, parts, chunks a part) of the tall product with parts: chunks of 128 k and K split so that the launch
    has about a workgroup a compute unit; where a part would then be longer than 1024 k (the down projection), chunks
    of 64 k and two workgroups a unit, up to 128 rows.  Measured at the 8B shapes, down projection: 30.3 us with
    chunks of 64 and 512 workgroups against 32.2 with chunks of 128 and 256 at 64 rows, 33.7 / 35.0 at 96, 37.1 / 42.3
    at 128, 60.7 / 52.0 at 208 (and the step at 160 rows 11.17 against 11.00 ms); o projection 12.5 / 11.0 at 64 rows,
    14.6 / 12.8 at 96."""
    n_tiles = -(-N // 128)

    def split(kc, wgs):
        chunks = -(-K // kc)
        kb = max(1, min(-(-wgs // n_tiles), chunks, TALL_MAX_PARTS))
        cpp = -(-chunks // kb)
        return kc, -(-chunks // cpp), cpp
    plan = split(128, 256)
    if plan[2] > 8 and M <= 128:
        plan = split(64, 512)
    return plan


def _gemm_tall(x: torch.Tensor, w: torch.Tensor, K: int, frag_w=None, plan: Optional[tuple] = None) -> torch.Tensor:
    """17 to 208 rows, result in float32 parts [P, M, N] split over K (see gemm_tall.hip)."""
    M, N = x.shape[0], w.shape[0]
    kc, kb, cpp = plan or _tall_plan(M, N, K)
    parts = torch.empty((kb, M, N), dtype=F32, device=x.device)
    fw = _frag_of(frag_w) if USE_FRAG else None
    if fw is not None:
        _run("ilm_gemm_tall", parts.data_ptr(), N, M * N, kb, cpp, kc, fw.data.data_ptr(), 0, M, N, K, x.data_ptr(), x.stride(0),
             1, _stream())
    else:
        _run("ilm_gemm_tall", parts.data_ptr(), N, M * N, kb, cpp, kc, w.data_ptr(), w.stride(0), M, N, K, x.data_ptr(),
             x.stride(0), 0, _stream())
    return parts


def gemm_tall_swiglu(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], frag_w=None, kc: int = 128) -> torch.Tensor:
    """silu(x Wg^T + bg) * (x Wu^T + bu) for 17 to 208 rows, W = [Wg; Wu] (see gemm_tall.hip)."""
    M, K = x.shape
    inter = w.shape[0] // 2
    act = torch.empty((M, inter), dtype=x.dtype, device=x.device)
    fw = _frag_of(frag_w) if USE_FRAG else None
    if fw is not None:
        _run("ilm_gemm_tall_swiglu", act.data_ptr(), act.stride(0), x.data_ptr(), x.stride(0), fw.data.data_ptr(), 0, _ptr(bias),
             M, inter, K, kc, 1, _stream())
    else:
        _run("ilm_gemm_tall_swiglu", act.data_ptr(), act.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
             _ptr(bias), M, inter, K, kc, 0, _stream())
    return act


USE_GATEUP_SWIGLU = os.environ.get("INFINILM_AMD_GATEUP_SWIGLU", "1") == "1"
# outputs from which the gate/up kernel with X in LDS is used (-1: 48 a compute unit; 0: always, as its tests do)
GATEUP_TALL_MIN_OUTPUTS = int(os.environ.get("INFINILM_AMD_GATEUP_TALL_MIN", "-1"))


# Rows up to which the projection that ends a branch takes the residual sum and the first half of the next
# norm into its epilogue (gemm_tail.hip); 0: never
TAIL_MAX_ROWS = int(os.environ.get("INFINILM_AMD_TAIL_ROWS", "16"))
TAIL_SS_ROWS = 32   # rows of a tile's record of partial sums of squares (ilm_gemm_tail_ss_rows())


def _mfma_operands_ok(x: torch.Tensor, w: torch.Tensor, K: int) -> bool:
    return (x.dtype == BF16 and w.dtype == BF16 and x.is_cuda and w.shape[1] == K and K % 8 == 0 and x.stride(1) == 1
            and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def tail_ok(rows: int, w: torch.Tensor, bias: Optional[torch.Tensor], norm_w: torch.Tensor, dtype: torch.dtype) -> bool:
    """Whether `gemm_tail` takes a product of `rows` rows with the weight w [N, K] (see there)."""
    N, K = w.shape
    return (not FORCE_BASIC and dtype == BF16 and w.dtype == BF16 and 0 < rows <= min(TAIL_MAX_ROWS, 32)
            and (K <= 4096 or (rows <= 16 and K <= 8192)) and K % 8 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0 and norm_w.shape == (N,) and norm_w.dtype in (BF16, F32) and norm_w.is_contiguous()
            and (bias is None or (bias.shape == (N,) and bias.dtype == BF16 and bias.is_contiguous())))


def gemm_tail(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], alpha: float, residual: torch.Tensor,
              norm_w: torch.Tensor):
    """The projection that ends a branch, with the residual sum and the first half of the norm after it
    in its epilogue: residual += alpha * (x w^T + bias) in place (float32 [M, N]); returns (xw, ss) with
    xw = bfloat16(residual * norm_w) [M, N], not yet divided by the rows' root mean square, and ss
    [ceil(N / 16), 32] partial sums of squares of the residual's rows, which the consumer of xw adds up
    (`gateup_swiglu_gemm(..., row_ss=ss, eps=...)`).  For what `tail_ok` accepts."""
    M, K = x.shape
    N = w.shape[0]
    _dev(x, w, bias, residual, norm_w)
    if not (tail_ok(M, w, bias, norm_w, x.dtype) and _mfma_operands_ok(x, w, K)):
        raise KernelError(f"gemm_tail does not take {tuple(x.shape)} x {tuple(w.shape)}^T")
    if residual.dtype != F32 or tuple(residual.shape) != (M, N) or residual.stride(1) != 1:
        raise KernelError("the residual stream is a float32 tensor with dense rows of the product's width")
    xw = torch.empty((M, N), dtype=BF16, device=x.device)
    ss = torch.empty((-(-N // 16), TAIL_SS_ROWS), dtype=F32, device=x.device)
    _run("ilm_gemm_tail", residual.data_ptr(), residual.stride(0), xw.data_ptr(), xw.stride(0), ss.data_ptr(), x.data_ptr(),
         x.stride(0), w.data_ptr(), w.stride(0), _ptr(bias), norm_w.data_ptr(), _dt(norm_w), float(alpha), M, N, K, _stream())
    return xw, ss


def gateup_resident_ok(rows: int, w: torch.Tensor) -> bool:
    """Whether the gate/up kernel that keeps X in registers takes `rows` rows with the weight w [2I, K]."""
    K = w.shape[1]
    return (USE_GATEUP_SWIGLU and not FORCE_BASIC and w.dtype == BF16 and _few_rows(rows, K) and K <= 8192 and K % 8 == 0
            and w.shape[0] % 2 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def gateup_swiglu_gemm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                       row_ss: Optional[torch.Tensor] = None, eps: float = 0.0, frag_w=None) -> Optional[torch.Tensor]:
    """silu(x Wg^T + bg) * (x Wu^T + bu) for few rows in bfloat16, W = [Wg; Wu]: the fused gate/up
    projection with the SwiGLU in its epilogue, [M, I] (up to 32 rows with X in registers; 17 to 208 with chunks
    of X in LDS where the outputs fill the chip).  None where no kernel applies (more rows, few outputs,
    float32): the caller then runs the projection and the activation.  `row_ss`: x is what `gemm_tail` left (residual * norm weight) and row_ss its
    partial sums of squares: the rows' division by sqrt(mean square + eps) happens in this kernel's
    epilogue (only the kernel with X in registers does that: `gateup_resident_ok`)."""
    M, K = x.shape
    resident = _few_rows(M, K) and K <= 8192
    if row_ss is not None:
        if not (resident and gateup_resident_ok(M, w) and _mfma_operands_ok(x, w, K) and row_ss.dtype == F32
                and row_ss.dim() == 2 and row_ss.shape[1] == TAIL_SS_ROWS and row_ss.is_contiguous() and row_ss.is_cuda):
            raise KernelError("a product with the norm's division in its epilogue needs the few-rows gate/up kernel")
    # (a workgroup takes 64 outputs: with fewer outputs than three quarters of the compute units have workgroups
    # the library is faster - measured with the kernel this one replaced, which cut alike: 2B-family shape, 5,760
    # outputs, 64 rows: 6.40 against 6.07 ms a step)
    tall_min = GATEUP_TALL_MIN_OUTPUTS if GATEUP_TALL_MIN_OUTPUTS >= 0 else 48 * _num_cus(x.device)
    # 17 to 112 rows, and up to 176 where the rows are no multiple of 32 (the vendor library's product is then slow):
    # chunks of X resident in LDS, two workgroups a compute unit (gemm_tall.hip).  Measured at the 8B shape: 48.1 us
    # against 52.9 (X in registers, two row groups) at 32 rows, 53.2 against 57.4 (X through LDS in steps of 256 k, one
    # workgroup a unit: the kernel it replaced) at 64; against the library's product and the activation kernel 57.7 / 66.2 at 96, 66.5 / 81.4 at
    # 112, 71.2 / 69.0 at 128, 76.1 / 85.2 at 144, 75.3 / 72.7 at 160, 82.8 / 90.1 at 176, 86.6 / 75.6 at 192, 90.4 / 83.0 at 208
    tall = (USE_TALL and row_ss is None and max(TALL_MIN_ROWS, 17) <= M <= TALL_MAX_ROWS
            and w.shape[0] // 2 >= tall_min and (M <= TALL_GATEUP_MAX_ROWS or (M % 32 != 0 and M <= 176)))
    if not (USE_GATEUP_SWIGLU and not FORCE_BASIC and x.dtype == BF16 and w.dtype == BF16 and x.is_cuda
            and (resident or tall) and K % 8 == 0 and w.shape[0] % 2 == 0 and w.shape[1] == K
            and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return None
    _dev(x, w, bias)
    I = w.shape[0] // 2
    if bias is not None and (bias.shape != (2 * I,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused gate/up projection")
    if tall:
        return gemm_tall_swiglu(x, w, bias, frag_w)
    out = torch.empty((M, I), dtype=BF16, device=x.device)
    _run("ilm_gemm_gateup_swiglu", out.data_ptr(), out.stride(0), x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0),
         _ptr(bias), M, I, K, _ptr(row_ss), 0 if row_ss is None else row_ss.shape[0], float(eps), _stream())
    return out


def swiglu_gemm(gate_up: torch.Tensor, w: torch.Tensor) -> Optional[torch.Tensor]:
    """(silu(gate) * up) w^T for at most 32 rows [gate | up] in bfloat16, in one kernel: float32 parts
    [P, M, N] for add_rmsnorm.  None when the shapes do not fit (the caller then runs the two kernels)."""
    M, two_k = gate_up.shape
    K = two_k // 2
    N = w.shape[0]
    # (above 32 rows the activation would be recomputed by every workgroup along N: the separate kernel
    # and the product with parts are faster, 38 against 42 us at 64 rows)
    ok = (gate_up.dtype == BF16 and w.dtype == BF16 and not FORCE_BASIC and USE_KSPLIT and M <= max(16, FEW_ROWS)
          and two_k % 2 == 0
          and w.shape[1] == K and K % 8 == 0 and gate_up.stride(1) == 1 and w.stride(1) == 1 and gate_up.stride(0) % 8 == 0
          and w.stride(0) % 8 == 0 and gate_up.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and gate_up.is_cuda)
    if not ok:
        return None
    kb = -(-K // KSPLIT_SPAN)
    parts = torch.empty((kb, M, N), dtype=F32, device=gate_up.device)
    _run("ilm_gemm_ksplit", parts.data_ptr(), _DT[F32], N, M * N, kb, w.data_ptr(), w.stride(0), None, 1.0,
         M, N, K, gate_up.data_ptr(), gate_up.stride(0), 1, _stream())
    return parts


_NUM_CUS: dict = {}


def _num_cus(device) -> int:
    """Compute units of the device (looked up once)."""
    cus = _NUM_CUS.get(device)
    if cus is None:
        cus = _NUM_CUS[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return cus


def bound_pages(need: int) -> int:
    """The block-table width a context of `need` pages is served with: 4, 6, 8, 12, 16, 24, ... (at
    most a third above the need).  The step function records one graph a width, and the attention
    kernels size their grids for it, so an eager step and a replayed one cut their keys alike."""
    width = 4
    while width < need:
        width = width * 3 // 2 if width & (width - 1) == 0 else width * 4 // 3
    return width


def bound_rows(rows: int) -> int:
    """The number of rows a decode step of `rows` requests is served with when it is recorded: 1, 2, 4, 8,
    16, 24, 32, 48, 64, 96, 128, 160, 208, 256, 384, 512, ... (the rest are rows of no request).  The sizes end
    where the products change kernels (16, 32, 64 rows; 208, the last size of the product with chunks of X in LDS), so a
    filled-up step runs the kernels the step itself would run and its recording equals the eager step."""
    for b in (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 160, 208, 256):
        if rows <= b:
            return b
    b = 256
    while b < rows:
        b = b * 3 // 2 if b & (b - 1) == 0 else b * 4 // 3
    return b


def attention_chunks(max_total_len: int, page: int, pairs: int, device) -> tuple:
    """(keys a chunk, chunks) of the chunked single-token attention for `pairs` = tokens x head groups.

    A chunk is a whole number of steps of ATT_STEP keys.  Few tokens: one step a chunk (latency
    counts, the chip is not full anyway).  Up to four steps as long as the launch still has a
    workgroup for every compute unit (fewer partial results to write and merge), and beyond that
    while it still has two for each.  Measured at the 8B head shape, 4096 keys, kernel + merge:
    8 tokens 17.0 us with 256 keys a chunk (128: 18.4, 512: 20.2); 16 tokens 22.4 with 512 (256:
    24.0); 32 tokens 34.3 with 512 (256: 40.0, 1024: 36.5); 64 tokens 57.5 with 1024 (512: 60.5).
    At most ATT_MAX_CHUNKS chunks (one token over 32,768 keys: 128 chunks of 256 keys 14.9 us, 64 of 512 18.1).  The length is first rounded up the way the step function rounds
    its graphs' block tables (`bound_pages`), so that an eager step and a replayed one cut alike."""
    bound = bound_pages(-(-max_total_len // page)) * page
    cus = _num_cus(device)
    steps = -(-bound // ATT_STEP)
    pairs = max(pairs, 1)
    workgroups = lambda per_chunk: pairs * -(-steps // per_chunk)
    per_chunk = 1
    for n in (2, 3, 4):
        if workgroups(n) >= cus:
            per_chunk = n
    while per_chunk >= 4 and 2 * per_chunk <= steps and workgroups(2 * per_chunk) >= 2 * cus:
        per_chunk *= 2
    # More workgroups than the chip holds at once (two a compute unit): they run in rounds, and a last round that is
    # nearly empty costs as much as a full one.  Among chunks of a quarter to twice that length take the one with the
    # least rounds x (steps a chunk + a workgroup's fixed cost, about three quarters of a step) + the chunks' merge.
    # Measured at the 8B head shape, 4096 keys, kernel + merge: 80 tokens 80.7 us with 512 keys a chunk (1024: 91.1),
    # 96 tokens 89.1 with 512 (1024: 95.9), 160 tokens 148.4 with 512 (2048: 170.4), 192 tokens 159.0 with 1024
    # (2048: 174.9); 160 tokens over 8192 keys 267.4 with 1024 (4096: 317.7).
    slots = 2 * cus
    if workgroups(per_chunk) > slots:
        def cost(n):
            return -(-workgroups(n) // slots) * (0.75 + n) + 0.15 * -(-steps // n)
        best = per_chunk
        for n in (per_chunk * 2, per_chunk // 2, per_chunk // 4):
            if 2 <= n <= steps and (cost(n), -n) < (cost(best), -best):
                best = n
        per_chunk = best
    while -(-steps // per_chunk) > ATT_MAX_CHUNKS:
        per_chunk += 1
    span = per_chunk * ATT_STEP
    return span, -(-max_total_len // span)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    seg_of_token: torch.Tensor, positions: torch.Tensor, nh: int, nkv: int, d: int,
                    scale: float, window: int = 0, max_total_len: Optional[int] = None,
                    tiles: Optional[torch.Tensor] = None, single_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of every token over its request's cached keys up to its own position.

    q: rows of T tokens in which head h lies at [h*d, (h+1)*d) (a view into the fused projection is
    fine); caches as the cache manager lays them out; block_tables [R, max_blocks]; `max_total_len`: an
    upper bound of position + 1 over the batch (the matrix-core kernel sizes its key chunks by it;
    without it the plain kernel runs).  `tiles` [n, 2] = (first row, count <= ATT_TILE_TOKENS) lists runs of
    consecutive tokens of one request and `single_rows` the remaining rows; without them every token
    is served on its own.  Returns [T, nh*d]."""
    _dev(q, k_cache, v_cache, block_tables, seg_of_token, positions)
    _i32(block_tables, "block_tables")
    _i32(seg_of_token, "seg_of_token")
    _i32(positions, "positions")
    T = q.shape[0]
    if q.stride(1) != 1 or q.shape[1] < nh * d:
        raise KernelError("q rows must be dense and hold all query heads")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError(f"cache dtype {k_cache.dtype} differs from the activations' {q.dtype}")
    page = _check_cache(k_cache, v_cache, nkv, d)
    if seg_of_token.numel() != T or positions.numel() != T or block_tables.dim() != 2:
        raise KernelError("per-token metadata does not match the number of tokens")
    out = torch.empty((T, nh * d), dtype=q.dtype, device=q.device)
    if (q.dtype == BF16 and not FORCE_BASIC and d % 16 == 0 and d <= 128 and page % 16 == 0 and q.stride(0) % 8 == 0
            and max_total_len is not None):
        n_single = T
        rows = None
        if tiles is not None and tiles.numel() > 0:
            # portions of prompts: tiles of consecutive tokens share their keys through LDS
            _i32(tiles, "tiles")
            _run("ilm_attn_tile", out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                 block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), tiles.data_ptr(),
                 tiles.numel() // 2, nh, nkv, d, page, block_tables.shape[1], q.stride(0), out.stride(0), float(scale),
                 int(window), _stream())
            if single_rows is None or single_rows.numel() == 0:
                return out
            _i32(single_rows, "single_rows")
            rows, n_single = single_rows, single_rows.numel()
        # (the tokens counted as the recorded steps round them, so that an eager step and a replayed one cut alike)
        span, nsplit = attention_chunks(int(max_total_len), page, bound_rows(n_single) * nkv * (-(-(nh // nkv) // 16)), q.device)
        ws_acc = ws_ml = None
        if nsplit > 1:
            # partial results of the rows served here (not of every token of the step)
            ws_acc = torch.empty((n_single * nh * nsplit * d,), dtype=F32, device=q.device)
            ws_ml = torch.empty((n_single * nh * nsplit * 2,), dtype=F32, device=q.device)
        _run("ilm_attn_mfma", out.data_ptr(), _ptr(ws_acc), _ptr(ws_ml), q.data_ptr(), k_cache.data_ptr(),
             v_cache.data_ptr(), block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), _ptr(rows),
             n_single, nh, nkv, d, page, block_tables.shape[1], q.stride(0), out.stride(0), float(scale), int(window),
             nsplit, span, _stream())
        return out
    bound = block_tables.shape[1] * page if max_total_len is None else min(int(max_total_len), block_tables.shape[1] * page)
    if (q.dtype == F32 and not FORCE_BASIC and d % 16 == 0 and d <= 256 and page % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0 and k_cache.data_ptr() % 16 == 0 and v_cache.data_ptr() % 16 == 0):
        # the 32-bit path: the group's heads side by side on the float matrix instruction.  Few tokens (decoding):
        # one wave a chunk of keys and a fold; many: one wave a token that walks its chunks.  The same bits.
        ws, nchunks = None, 1
        waves = T * nkv * -(-(nh // nkv) // 16)
        if F32_ATTN_SPLIT and waves <= F32_ATTN_SPLIT_WAVES and bound > F32_ATTN_CHUNK:
            nchunks = -(-bound // F32_ATTN_CHUNK)
            ws = torch.empty((T * nh * nchunks * (d + 4),), dtype=F32, device=q.device)
        _run("ilm_attn_f32", out.data_ptr(), _ptr(ws), nchunks, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
             block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), T, nh, nkv, d, page,
             block_tables.shape[1], q.stride(0), out.stride(0), float(scale), int(window), _stream())
        return out
    # The plain kernel.  Few tokens over long contexts (decoding): one wave a chunk of keys and a fold of the
    # partial results, instead of one wave a head; the bits are the same (see attn_basic.hip).
    ws, nchunks = None, 1
    if BASIC_SPLIT and T * nh <= BASIC_SPLIT_WAVES and bound > BASIC_CHUNK:
        nchunks = -(-bound // BASIC_CHUNK)
        ws = torch.empty((T * nh * nchunks * (d + 2),), dtype=F32, device=q.device)
    _run("ilm_attn_basic", out.data_ptr(), _ptr(ws), nchunks, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         block_tables.data_ptr(), seg_of_token.data_ptr(), positions.data_ptr(), T, nh, nkv, d, page, block_tables.shape[1],
         q.stride(0), out.stride(0), float(scale), int(window), _dt(q), _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    _dev(logits)
    if logits.dtype != F32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax takes float32 rows")
    n, V = logits.shape
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _run("ilm_argmax", out.data_ptr(), logits.data_ptr(), n, V, logits.stride(0), _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor) -> torch.Tensor:
    """One token a row; per-row temperature (float32), top_k (int32), top_p (float32), u in [0,1)."""
    _dev(logits, temperature, top_k, top_p, uniform)
    if logits.dtype != F32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample takes float32 rows")
    n, V = logits.shape
    _i32(top_k, "top_k")
    for t, nm in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if t.dtype != F32 or t.numel() != n or not t.is_contiguous():
            raise KernelError(f"{nm} must be float32 with one entry a row")
    if top_k.numel() != n:
        raise KernelError("top_k must have one entry a row")
    out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _run("ilm_sample", out.data_ptr(), logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
         uniform.data_ptr(), n, V, logits.stride(0), _stream())
    return out


# ---- operands in fragment order (csrc/frag.h): the products of a decode step ------------------------------
FRAG_MAX_ROWS = 64    # most rows of X the fragment-order products take
FRAG_SS_ROWS = 64     # rows of a tile's record of partial sums of squares (ilm_gemm_frag_ss_rows())
USE_FRAG = os.environ.get("INFINILM_AMD_FRAG", "1") == "1" and not FORCE_BASIC
FRAG_TILES = int(os.environ.get("INFINILM_AMD_FRAG_TILES", "2"))   # tiles of W a workgroup (2 or 4)


class FragRows:
    """Activations [rows, width] in bfloat16, stored in fragment order (`data`: a flat int32 buffer)."""
    __slots__ = ("data", "rows", "width")

    def __init__(self, data: torch.Tensor, rows: int, width: int):
        self.data, self.rows, self.width = data, int(rows), int(width)

    @property
    def shape(self):
        return (self.rows, self.width)

    @property
    def dtype(self):
        return BF16

    @property
    def device(self):
        return self.data.device


def frag_rows_empty(rows: int, width: int, device) -> FragRows:
    """An uninitialised fragment-order buffer for [rows, width]; the k beyond the width (up to a multiple of 32)
    are zeros, as the products need them."""
    groups, steps = -(-rows // 16), -(-width // 32)
    if width % 32:
        data = torch.zeros((steps * groups * 64 * 4,), dtype=torch.int32, device=device)
    else:
        data = torch.empty((steps * groups * 64 * 4,), dtype=torch.int32, device=device)
    return FragRows(data, rows, width)


def to_frag(x: torch.Tensor) -> FragRows:
    """Plain bfloat16 rows into fragment order (a kernel of its own: for producers that have no such store)."""
    _dev(x)
    M, K = x.shape
    if x.dtype != BF16 or x.stride(1) != 1 or K % 8 or x.stride(0) % 8 or x.data_ptr() % 16:
        raise KernelError("fragment order takes bfloat16 rows of a multiple of 8 elements, 16-byte aligned")
    out = FragRows(torch.empty((-(-K // 32) * -(-M // 16) * 64 * 4,), dtype=torch.int32, device=x.device), M, K)
    _run("ilm_frag_pack_rows", out.data.data_ptr(), x.data_ptr(), M, K, x.stride(0), _stream())
    return out


def from_frag(f: FragRows) -> torch.Tensor:
    out = torch.empty((f.rows, f.width), dtype=BF16, device=f.data.device)
    _run("ilm_frag_unpack_rows", out.data_ptr(), f.data.data_ptr(), f.rows, f.width, f.width, _stream())
    return out


class FragWeight:
    """A weight [N, K] in fragment order: tiles of 16 rows in the order `rows` names (None: W's own), padded to a
    multiple of 4 tiles; `tiles` counts the real ones."""
    __slots__ = ("data", "N", "K", "tiles", "kind")

    def __init__(self, data, N, K, tiles, kind):
        self.data, self.N, self.K, self.tiles, self.kind = data, N, K, tiles, kind


def frag_weight_ok(w: torch.Tensor) -> bool:
    return (USE_FRAG and w.is_cuda and w.dtype == BF16 and w.dim() == 2 and w.shape[1] % 8 == 0 and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def pack_weight(w: torch.Tensor, kind: str = "plain", **layout) -> FragWeight:
    """`kind`: "plain" (tiles of consecutive rows), "gate_up" (w = [Wg; Wu]: tile pairs (gate rows 16p.., up rows 16p..)),
    "qkv" (nh, nkv, d given: tile pairs (first rows, second rows) of 16 rotation pairs; pair p = head slot p // (d/2),
    dim p % (d/2))."""
    if not frag_weight_ok(w):
        raise KernelError("fragment order takes a bfloat16 weight with rows of a multiple of 8 elements, 16-byte aligned")
    N, K = w.shape
    rows = None
    alloc_to = 4
    if kind == "plain":
        tiles = -(-N // 16)
    elif kind == "gate_up":
        I = N // 2
        it = -(-I // 16)
        idx = torch.arange(it * 16, dtype=torch.int64).view(it, 16)
        g = torch.where(idx < I, idx, torch.full_like(idx, -1))
        u = torch.where(idx < I, idx + I, torch.full_like(idx, -1))
        rows = torch.stack([g, u], dim=1).reshape(-1)
        tiles = 2 * it
    elif kind == "gate_up8":   # tiles of 8 gate rows and the 8 up rows of the same outputs
        I = N // 2
        it = -(-I // 8)
        idx = torch.arange(it * 8, dtype=torch.int64).view(it, 8)
        g = torch.where(idx < I, idx, torch.full_like(idx, -1))
        u = torch.where(idx < I, idx + I, torch.full_like(idx, -1))
        rows = torch.cat([g, u], dim=1).reshape(-1)
        tiles = it
        alloc_to = 8   # a workgroup of the kernel that reads it takes 8 tiles
    elif kind == "qkv":
        nh, nkv, d = layout["nh"], layout["nkv"], layout["d"]
        half = d // 2
        pairs = (nh + 2 * nkv) * half
        pt = -(-pairs // 16)
        p = torch.arange(pt * 16, dtype=torch.int64).view(pt, 16)
        first = (p // half) * d + p % half
        a = torch.where(p < pairs, first, torch.full_like(p, -1))
        b = torch.where(p < pairs, first + half, torch.full_like(p, -1))
        rows = torch.stack([a, b], dim=1).reshape(-1)
        tiles = 2 * pt
    else:
        raise KernelError(f"unknown fragment layout {kind!r}")
    alloc = -(-tiles // alloc_to) * alloc_to
    steps = -(-K // 32)
    data = torch.zeros((alloc * steps * 64 * 4,), dtype=torch.int32, device=w.device)
    rows_dev = None
    if rows is not None:
        rows_dev = rows.to(torch.int32).to(w.device)
    _run("ilm_frag_pack_weight", data.data_ptr(), w.data_ptr(), _ptr(rows_dev), N, K, w.stride(0), tiles, _stream())
    return FragWeight(data, N, K, tiles, kind)


# Rows from which the q/k/v projection of a decode step takes its operands in fragment order (measured at the 8B
# shape: 12.7 against 17.3 us at 32 rows, 16.2 against 22.5 us for the vendor library's product and the rotation
# kernel at 64; up to 16 rows the kernel that keeps X in registers is as fast)
FRAG_QKV_MIN_ROWS = int(os.environ.get("INFINILM_AMD_FRAG_QKV_MIN_ROWS", "17"))


def qkv_frag_ok(rows: int, w: torch.Tensor, d: int, rd: int, width: int) -> bool:
    """Whether the fused q/k/v projection takes `rows` rows in fragment order (see `gemm_frag_rope`)."""
    return (FRAG_QKV_MIN_ROWS <= rows <= FRAG_MAX_ROWS and frag_weight_ok(w) and rd == d and d % 32 == 0 and width % 8 == 0
            and USE_QKV_ROPE)


def _frag_x(x: FragRows, fw: FragWeight) -> None:
    if not isinstance(x, FragRows) or x.width != fw.K or x.rows > FRAG_MAX_ROWS:
        raise KernelError(f"fragment-order product: X {getattr(x, 'shape', None)} does not fit W [{fw.N}, {fw.K}] "
                          f"(at most {FRAG_MAX_ROWS} rows)")


def gemm_frag(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor] = None, alpha: float = 1.0,
              out: str = "bf16", parts: int = 1):
    """alpha (x W^T + bias) of up to 64 rows.  `out`: "bf16" or "f32" rows [M, N]; "parts": float32 [parts, M, N] of a
    K split in `parts` ranges (for add_rmsnorm); "frag": bfloat16 in fragment order."""
    _frag_x(x, fw)
    M, N, K = x.rows, fw.N, fw.K
    steps = -(-K // 32)
    spp = 0
    if out == "parts":
        spp = -(-steps // max(parts, 1))
        spp = -(-spp // 8) * 8 if spp > 8 else spp
        parts = -(-steps // spp)
        res = torch.empty((parts, M, N), dtype=F32, device=x.device)
        kind, ldc, target = 1, N, res
    elif out == "f32":
        res = torch.empty((M, N), dtype=F32, device=x.device)
        kind, ldc, target = 1, N, res
    elif out == "bf16":
        res = torch.empty((M, N), dtype=BF16, device=x.device)
        kind, ldc, target = 0, N, res
    else:
        res = frag_rows_empty(M, N, x.device)
        kind, ldc, target = 2, N, res.data
    if bias is not None and (bias.shape != (N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the product")
    _run("ilm_gemm_frag", target.data_ptr(), ldc, M * N, kind, x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), M, N, K,
         spp, float(alpha), FRAG_TILES, _stream())
    return res


def gemm_frag_swiglu(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor] = None,
                     row_ss: Optional[torch.Tensor] = None, norm_width: int = 0, eps: float = 0.0) -> FragRows:
    """silu(x Wg^T + bg) * (x Wu^T + bu) in fragment order; `row_ss`: x is what `gemm_frag_tail` left and the rows'
    division by sqrt(mean square + eps) over `norm_width` happens here."""
    _frag_x(x, fw)
    if fw.kind != "gate_up":
        raise KernelError("the SwiGLU epilogue needs a weight packed as gate_up")
    I = fw.N // 2
    if bias is not None and (bias.shape != (2 * I,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused gate/up projection")
    if row_ss is not None and (row_ss.dtype != F32 or row_ss.dim() != 2 or row_ss.shape[1] != FRAG_SS_ROWS or not row_ss.is_contiguous()):
        raise KernelError("partial sums of squares must be float32 [tiles, 64]")
    act = frag_rows_empty(x.rows, I, x.device)
    _run("ilm_gemm_frag_swiglu", act.data.data_ptr(), x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), x.rows, I, fw.K,
         _ptr(row_ss), 0 if row_ss is None else row_ss.shape[0], int(norm_width), float(eps), FRAG_TILES, _stream())
    return act


def gemm_frag_rope(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor], positions: torch.Tensor, cos: torch.Tensor,
                   sin: torch.Tensor, k_cache, v_cache, slots, nh: int, nkv: int, d: int) -> torch.Tensor:
    """The fused q/k/v projection with rotation and cache write; returns the rotated q [M, nh*d]."""
    _frag_x(x, fw)
    if fw.kind != "qkv" or fw.N != (nh + 2 * nkv) * d or d % 32:
        raise KernelError("the rotation epilogue needs a weight packed as qkv with heads in steps of 32")
    M = x.rows
    _i32(positions, "positions")
    if positions.numel() != M:
        raise KernelError("positions must have one entry a row")
    if cos.dtype != F32 or sin.dtype != F32 or cos.shape != sin.shape or cos.shape[1] != d // 2 \
            or not cos.is_contiguous() or not sin.is_contiguous():
        raise KernelError(f"rotation tables must be float32 [positions, {d // 2}], got {tuple(cos.shape)}")
    if bias is not None and (bias.shape != (fw.N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the fused projection")
    page = 0
    if slots is not None:
        _i32(slots, "slots")
        if k_cache is None or v_cache is None or k_cache.dtype != BF16 or v_cache.dtype != BF16:
            raise KernelError("cache tensors missing or of another dtype than the activations")
        page = _check_cache(k_cache, v_cache, nkv, d)
    q = torch.empty((M, nh * d), dtype=BF16, device=x.device)
    _run("ilm_gemm_frag_rope", q.data_ptr(), q.stride(0), x.data.data_ptr(), fw.data.data_ptr(), _ptr(bias), M, fw.K,
         positions.data_ptr(), cos.data_ptr(), sin.data_ptr(), _ptr(k_cache) if slots is not None else None,
         _ptr(v_cache) if slots is not None else None, _ptr(slots), nh, nkv, d, page, _stream())
    return q


def gemm_frag_tail(x: FragRows, fw: FragWeight, bias: Optional[torch.Tensor], alpha: float, residual: torch.Tensor,
                   norm_w: torch.Tensor):
    """residual += alpha (x W^T + bias) in place; returns (xw, ss): xw = bfloat16(residual * norm_w) in fragment order,
    ss [ceil(N / 16), 64] partial sums of squares of the residual's rows."""
    _frag_x(x, fw)
    M, N = x.rows, fw.N
    if fw.kind != "plain":
        raise KernelError("the tail epilogue needs a weight packed plainly")
    if residual.dtype != F32 or tuple(residual.shape) != (M, N) or residual.stride(1) != 1:
        raise KernelError("the residual stream is a float32 tensor with dense rows of the product's width")
    if norm_w.shape != (N,) or norm_w.dtype not in (BF16, F32) or not norm_w.is_contiguous():
        raise KernelError("the norm's weight does not fit")
    if bias is not None and (bias.shape != (N,) or bias.dtype != BF16 or not bias.is_contiguous()):
        raise KernelError("bias does not fit the product")
    xw = frag_rows_empty(M, N, x.device)
    ss = torch.empty((-(-N // 16), FRAG_SS_ROWS), dtype=F32, device=x.device)
    _run("ilm_gemm_frag_tail", residual.data_ptr(), residual.stride(0), xw.data.data_ptr(), ss.data_ptr(), x.data.data_ptr(),
         fw.data.data_ptr(), _ptr(bias), norm_w.data_ptr(), 1 if norm_w.dtype == F32 else 0, float(alpha), M, N, fw.K,
         FRAG_TILES, _stream())
    return xw, ss
