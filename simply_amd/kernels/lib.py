"""Loads the gfx950 kernel library and declares its C entry points.

There is no fallback: if the library is missing and cannot be built, or if an
entry point refuses its arguments, an exception is raised.
"""
from __future__ import annotations

import ctypes
import sys
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_uint32, c_void_p

from . import build as _build


class KernelError(RuntimeError):
    pass


_lock = threading.Lock()
_lib: ctypes.CDLL | None = None
_path: str | None = None

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float
_SIGNATURES = {
    "sa_embed": [_P, _I, _P, _P, _I, _I, _I, _F, _I, _P],
    "sa_rmsnorm": [_P, _I, _L, _P, _I, _P, _I, _L, _I, _I, _F, _I, _P],
    "sa_add_rmsnorm": [_P, _I, _P, _I, _F, _I, _P, _P, _I, _F, _I, _P, _I, _I, _I, _P],
    "sa_add_rmsnorm_rows": [_P, _I, _P, _I, _F, _I, _P, _P, _I, _F, _I, _P, _I, _P, _I, _I, _P],
    "sa_decode_advance_slots": [_I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _I, _P, _P, _P, _I, _P],
    "sa_rope_cache_write": [_P, _I, _L, _P, _P, _F, _F, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    "sa_rope_cache_write_planes": [_P, _I, _P, _L, _P, _P, _F, _F, _P, _P, _P, _I, _I, _I, _I, _I, _P],
    "sa_rope": [_P, _I, _L, _P, _P, _F, _F, _I, _I, _I, _P],
    "sa_gather_rows": [_P, _I, _P, _P, _I, _I, _I, _P],
    "sa_fill_u32": [_P, c_uint32, _L, _P],
    "sa_decode_advance": [_I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _P],
    "sa_decode_slots": [_I, _P, _P, _P, _I, _I, _P, _P],
    "sa_gemm": [_P, _I, _L, _P, _P, _I, _P, _I, _L, _I, _I, _I, _I, _F, _I, _I, _I, _P, _L, _P],
    "sa_gemm_planes": [_P, _I, _L, _P, _P, _I, _P, _I, _L, _I, _I, _I, _I, _F, _I, _I, _I, _P, _L, _P, _P],
    "sa_sum_planes": [_P, _I, _P, _I, _L, _I, _I, _P],
    "sa_add_rmsnorm_planes": [_P, _I, _P, _I, _F, _I, _P, _P, _I, _F, _I, _P, _I, _I, _I, _P],
    "sa_paged_attention": [_P, _I, _L, _P, _P, _P, _I, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "sa_paged_attention_decode": [_P, _L, _P, _P, _P, _I, _P, _I, _I, _P, _L, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P, _L,
                                  _P],
    "sa_paged_attention_prefill": [_P, _L, _P, _P, _P, _I, _P, _I, _I, _P, _L, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P, _L,
                                   _P],
    "sa_gemm_normed": [_P, _P, _P, _P, _I, _F, _I, _P, _I, _F, _I, _P, _P, _I, _L, _I, _I, _I, _I, _F, _P],
    "sa_gemm_normed_takes": [_I, _I, _I],
    "sa_gemm_normed_pays": [_I, _I, _I],
    "sa_gemm_normed_max_rows": [],
    "sa_paged_attention_prefill_group": [],
    "sa_paged_attention_decode_takes": [_I, _I, _I, _I, _I, _L, _P],
    "sa_gemm_normed_rotary": [_P, _P, _P, _P, _I, _F, _I, _P, _I, _F, _I, _P, _P, _I, _L, _I, _I, _P, _P, _F, _F, _P, _P,
                              _P, _I, _I, _I, _I, _P],
    "sa_score": [_P, _L, _I, _I, _P, _P, _P, _P, _P, _P],
    "sa_probe_hbm_read": [_P, _L, _P, _P, _P],
    "sa_probe_mfma": [_P, _I, _I, _P, _P],
    "sa_sample": [_P, _L, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P, _L, _P],
}


def library_path() -> str | None:
    return _path


def load() -> ctypes.CDLL:
    """The loaded library; built first if no built library is found."""
    global _lib, _path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        import torch  # noqa: F401  (loads the HIP runtime that the library links against)

        path = _build.find_library()
        if path is None:
            print("[simply_amd] no built kernel library found: compiling the gfx950 kernels (about a minute)",
                  file=sys.stderr, flush=True)
            path = _build.build(verbose=True)
        elif _build.is_stale(path):
            print(f"[simply_amd] warning: {path} was built from other sources than those in the tree; "
                  "run `python -m simply_amd.kernels.build`", file=sys.stderr, flush=True)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"the kernel library {path} could not be loaded: {e}") from e
        lib.sa_last_error.restype = c_char_p
        lib.sa_last_error.argtypes = []
        lib.sa_version.restype = c_int
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = c_int
        lib.sa_gemm_plan.argtypes = [_I, _I, _I, _I, _I, _L, _P]
        lib.sa_gemm_plan.restype = c_int
        lib.sa_philox4x32_10.argtypes = [_P, _P, _P]
        lib.sa_philox4x32_10.restype = None
        _lib, _path = lib, path
        return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.sa_last_error().decode(errors="replace"))
