"""Loads the compiled kernel library and declares its C entry points.

The library shares the process's HIP runtime with PyTorch (PyTorch is imported first, so the
runtime it ships is the one the dynamic linker binds), which makes PyTorch's streams and device
pointers valid arguments.  There is no fallback: without the library, or without a GPU at call
time, the kernels raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p
from typing import Optional

_lib: Optional[ctypes.CDLL] = None

_P = c_void_p
_I = c_int
_F = c_float
_L = c_long

_SIGNATURES = {
    "ilm_embed": [_P, _P, _P, _I, _I, _I, _F, _I, _P],
    "ilm_add_rmsnorm": [_P, _P, _P, _P, _I, _I, _F, _F, _I, _I, _I, _I, _L, _I, _P],
    "ilm_gemm_ksplit": [_P, _I, _I, _L, _I, _P, _I, _P, _F, _I, _I, _I, _P, _I, _I, _P],
    "ilm_rope_kvwrite": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "ilm_swiglu": [_P, _P, _I, _I, _I, _I, _P],
    "ilm_gather_rows": [_P, _P, _P, _I, _I, _I, _P],
    "ilm_scale_rows": [_P, _I, _I, _I, _F, _P],
    "ilm_gemm_gateup_swiglu": [_P, _I, _P, _I, _P, _I, _P, _I, _I, _I, _P, _I, _F, _P],
    "ilm_gemm_tail": [_P, _I, _P, _I, _P, _P, _I, _P, _I, _P, _P, _I, _F, _I, _I, _I, _P],
    "ilm_gemm_rows64": [_P, _I, _L, _I, _P, _I, _I, _I, _I, _P, _I, _I, _P],
    "ilm_gemm_tall": [_P, _I, _L, _I, _I, _I, _P, _I, _I, _I, _I, _P, _I, _I, _P],
    "ilm_gemm_tall_swiglu": [_P, _I, _P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _P],
    "ilm_gemm_qkv_rope": [_P, _I, _P, _I, _P, _I, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "ilm_frag_pack_weight": [_P, _P, _P, _I, _I, _I, _I, _P],
    "ilm_frag_pack_rows": [_P, _P, _I, _I, _I, _P],
    "ilm_frag_unpack_rows": [_P, _P, _I, _I, _I, _P],
    "ilm_gemm_frag": [_P, _I, _L, _I, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P],
    "ilm_gemm_frag_swiglu": [_P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _F, _I, _P],
    "ilm_gemm_frag_rope": [_P, _I, _P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "ilm_gemm_frag_tail": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _F, _I, _I, _I, _I, _P],
    "ilm_gemm_f32_skinny": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P],
    "ilm_gemm_f32_tile": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P],
    "ilm_attn_f32": [_P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "ilm_gemm_basic": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ilm_attn_basic": [_P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ilm_gemm_skinny": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ilm_attn_mfma": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P],
    "ilm_attn_mfma_static": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P],
    "ilm_attn_tile": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "ilm_argmax": [_P, _P, _I, _I, _I, _P],
    "ilm_sample": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
}


def _check_single_hip_runtime() -> None:
    try:
        with open("/proc/self/maps") as fh:
            libs = {line.split()[-1] for line in fh if "libamdhip64" in line}
    except OSError:
        return
    real = {__import__("os").path.realpath(p) for p in libs}
    if len(real) > 1:
        raise RuntimeError("infinilm_amd: two HIP runtimes are loaded in this process (" + ", ".join(sorted(real))
                           + "); the kernel library and PyTorch must share one")


def load(verbose: bool = True) -> ctypes.CDLL:
    """The library, compiled first if no up-to-date build exists."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (binds PyTorch's HIP runtime before ours is resolved)
    from . import build as _build

    path = _build.ensure_built(verbose=verbose)
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    _check_single_hip_runtime()
    lib.ilm_last_error.restype = ctypes.c_char_p
    lib.ilm_last_error.argtypes = []
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise RuntimeError(f"infinilm_amd: {path} lacks the entry point {name}; rebuild it "
                               "(python -c 'import __graft_entry__ as g; g.build()')")
        fn.argtypes = args
        fn.restype = c_int
    lib.ilm_attn_static_init.restype = c_int
    lib.ilm_attn_static_init.argtypes = []
    lib.ilm_attn_static_scratch_floats.restype = c_long
    lib.ilm_attn_static_scratch_floats.argtypes = []
    _lib = lib
    return lib


def last_error() -> str:
    return load().ilm_last_error().decode(errors="replace")
