"""Builds the gfx950 kernel library with hipcc.

`python -m simply_amd.kernels.build` compiles every source under
`simply_amd/csrc/` and links `libsimply_amd_gfx950.so` beside this file.  The
library has no dependency on Python or torch: it exports C entry points that take
device pointers and a stream.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

ARCH = "gfx950"
LIB_NAME = f"libsimply_amd_{ARCH}.so"
HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed 32-bit float instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _say(msg: str) -> None:
    print(f"[simply_amd build] {msg}", file=sys.stderr, flush=True)


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_digest() -> str:
    h = hashlib.sha256()
    for f in sorted(os.listdir(CSRC)):
        if f.endswith((".hip", ".h")):
            h.update(f.encode())
            with open(os.path.join(CSRC, f), "rb") as fh:
                h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise RuntimeError("hipcc was not found (PATH, $HIPCC, /opt/rocm/bin): the gfx950 kernels cannot be built")


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        with tempfile.NamedTemporaryFile(dir=d):
            pass
        return True
    except OSError:
        return False


def candidate_dirs() -> list[str]:
    """Where the library may lie: beside this file, else a per-user folder in the
    temporary directory (for a checkout that its user cannot write)."""
    out = []
    env = os.environ.get("SIMPLY_AMD_LIB_DIR")
    if env:
        out.append(env)
    out.append(HERE)
    out.append(os.path.join(tempfile.gettempdir(), f"simply_amd_{os.getuid()}_{source_digest()}"))
    return out


def find_library() -> str | None:
    for d in candidate_dirs():
        p = os.path.join(d, LIB_NAME)
        if os.path.isfile(p):
            return p
    return None


def _run(cmd: list[str], what: str) -> None:
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a HOME for its caches
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr, flush=True)


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compiles all sources (always) and returns the path of the linked library."""
    hipcc = find_hipcc()
    out_dir = next((d for d in candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library: " + ", ".join(candidate_dirs()))
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, (os.cpu_count() or 2))))
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(srcs)} HIP sources for {ARCH} with {jobs} jobs -> {out_dir}")

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        t = time.time()
        _run([hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj], f"compiling {os.path.basename(src)}")
        if verbose:
            _say(f"  {os.path.basename(src)} done in {time.time() - t:.1f} s ({time.time() - t0:.0f} s since start)")
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp], "linking")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, LIB_NAME + ".digest"), "w") as f:
        f.write(source_digest())
    if verbose:
        _say(f"linked {lib} in {time.time() - t0:.1f} s")
    return lib


def is_stale(lib: str) -> bool:
    try:
        with open(lib + ".digest") as f:
            return f.read().strip() != source_digest()
    except OSError:
        return False


if __name__ == "__main__":
    print(build())
