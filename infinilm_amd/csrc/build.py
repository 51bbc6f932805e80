"""Compiles the HIP sources of this folder for gfx950 into one shared library.

`hipcc` is called directly (no header of a tensor library is needed: the entry points take raw
device pointers and a stream), each source in its own process, then one link.  The library lies in
`_build/` beside the sources when that folder can be written, else in a per-user folder under the
system's temporary folder.  A digest of the sources and flags is stored beside it; a library whose
digest does not match is not loaded.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libinfinilm_hip.so"
ARCH = "gfx950"

# `-packed-fp32-ops` switched off: the compiler then makes no packed float32 instructions
# (v_pk_add_f32, v_pk_mul_f32, v_pk_fma_f32) out of scalar or float2 code; some of their forms have
# given wrong results on this hardware, now and then and without an error.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def digest() -> str:
    h = hashlib.sha256()
    for f in sources() + _headers():
        h.update(f.encode())
        with open(os.path.join(HERE, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:24]


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _candidate_dirs() -> List[str]:
    dirs = [os.path.join(HERE, "_build")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"infinilm_amd_build_{os.getuid()}"))
    return dirs


def _writable_dir() -> str:
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w") as fh:
                fh.write("x")
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("infinilm_amd: no writable folder for the kernel build: tried " + ", ".join(_candidate_dirs()))


def built_library() -> Optional[str]:
    """Path of an up-to-date library, or None."""
    want = digest()
    for d in _candidate_dirs():
        lib = os.path.join(d, LIB_NAME)
        tag = os.path.join(d, LIB_NAME + ".digest")
        if os.path.isfile(lib) and os.path.isfile(tag):
            try:
                with open(tag) as fh:
                    if fh.read().strip() == want:
                        return lib
            except OSError:
                pass
    return None


def _say(msg: str) -> None:
    print(f"[infinilm_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every source and link; returns the library's path.  Prints a line now and then."""
    hipcc = _hipcc()
    if hipcc is None:
        raise RuntimeError("infinilm_amd: hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                           "the HIP kernels cannot be compiled")
    out_dir = _writable_dir()
    srcs = sources()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)  # hipcc must not depend on a user's home
    if not env.get("HOME"):
        env["HOME"] = out_dir
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    max_par = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0") or 0) or (os.cpu_count() or 4), 16))
    pending = list(srcs)
    running = []
    objs = []
    last = time.time()
    while pending or running:
        while pending and len(running) < max_par:
            s = pending.pop(0)
            obj = os.path.join(out_dir, s[:-4] + f".{os.getpid()}.o")
            cmd = [hipcc] + HIPCC_FLAGS + ["-I", HERE, "-c", os.path.join(HERE, s), "-o", obj]
            p = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
            running.append((s, obj, p))
        still = []
        for s, obj, p in running:
            rc = p.poll()
            if rc is None:
                still.append((s, obj, p))
                continue
            out = p.stdout.read().decode(errors="replace")
            if rc != 0:
                for _, _, q in running:
                    if q is not p and q.poll() is None:
                        q.kill()
                raise RuntimeError(f"infinilm_amd: hipcc failed on {s}:\n{out}")
            objs.append(obj)
            if verbose:
                _say(f"compiled {s} ({time.time() - t0:.0f} s)")
                last = time.time()
        running = still
        if running:
            time.sleep(0.2)
            if verbose and time.time() - last > 10:
                _say("still compiling " + ", ".join(s for s, _, _ in running) + f" ({time.time() - t0:.0f} s)")
                last = time.time()
    tmp_lib = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc"] + sorted(objs) + ["-o", tmp_lib]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=out_dir)
    if r.returncode != 0:
        raise RuntimeError("infinilm_amd: link failed:\n" + r.stdout.decode(errors="replace"))
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(tmp_lib, lib)
    with open(lib + ".digest", "w") as fh:
        fh.write(digest())
    for o in objs:
        try:
            os.remove(o)
        except OSError:
            pass
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def ensure_built(verbose: bool = True) -> str:
    """The library's path; compiles only when no up-to-date library exists."""
    lib = built_library()
    if lib is not None:
        return lib
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
