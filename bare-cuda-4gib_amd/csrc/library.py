"""Loads ``libbc4g.so`` through ctypes and declares its entry points."""
from __future__ import annotations

import ctypes
import sys
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Optional

from ..errors import KernelError
from . import build as _build
from .profile import profiler

_P = c_void_p
_I = c_int
_F = c_float

# name -> argument types (every function returns int status, except where noted)
_SIGNATURES = {
    "bc4g_embed_gather": [_P, _I, _P, _P, _I, _I, _I, _P],
    "bc4g_rmsnorm": [_P, _P, _P, _I, _P, _I, _I, _I, _F, _P],
    "bc4g_rmsnorm_sum": [_P, _P, _I, _P, _I, _P, _I, _I, _I, _F, _P],
    "bc4g_gemm_mfma_parts": [_P, _P, _I, _P, _I, _I, _I, _I, _P],
    "bc4g_gemm_mfma_swiglu_scaled": [_P, _P, _I, _I, _F, _P, _I, _P, _I, _I, _I, _P],
    "bc4g_gemm_generic": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _P],
    "bc4g_swiglu": [_P, _P, _I, _I, _I, _I, _P],
    "bc4g_rope_table": [_P, _P, _I, _I, _F, _P],
    "bc4g_rope_kv_write_blocks": [_P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "bc4g_rope_kv_write": [_P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _P],
    "bc4g_attention_generic": [_P, _I, _P, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "bc4g_argmax": [_P, _P, _P, _P, _I, _I, _P],
    "bc4g_sample": [_P, _P, _P, _P, _I, _I, _P],
    "bc4g_sample_filtered": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _P],
    "bc4g_argmax_static": [_P, _P, _I, _I, _P],
    "bc4g_probe_read": [_P, c_long, _P, _I, _P],
    "bc4g_probe_mfma": [_P, _I, _P, _I, _P],
    "bc4g_gemm_skinny": [_P, _P, _P, _I, _I, _I, _I, _P],
    "bc4g_gemm_mfma": [_P, _P, _I, _P, _I, _I, _I, _I, _P],
    "bc4g_gemm_mfma_tile": [_P, _P, _I, _I, _I, _I, _P, _P],
    "bc4g_gemm_skinny_normed": [_P, _P, _P, _I, _F, _P, _P, _I, _I, _I, _I, _P],
    "bc4g_attention_mfma": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _P, _I, _P, _I, _P, _P],
    "bc4g_gemm_mfma_qkv": [_P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "bc4g_gemm_skinny_qkv": [_P, _P, _I, _F, _P, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "bc4g_gemm_skinny_emit": [_P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _P],
    "bc4g_gemm_skinny_prenormed": [_P, _P, _I, _I, _F, _P, _P, _I, _I, _I, _I, _P],
}

_lib: Optional[ctypes.CDLL] = None


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """The kernel library; compiled first if it has never been built.

    Fails loudly (KernelError) if it cannot be had: there is no other
    implementation of the kernels to fall back to.
    """
    global _lib
    if _lib is not None:
        return _lib
    if not _build.is_built():
        if not build_if_missing:
            raise KernelError(f"{_build.LIB_PATH} is not built; run __graft_entry__.build()")
        _build.build(verbose=True)
    elif _build.is_stale():
        # A library built from other sources than those beside it would be called with the wrong
        # arguments (entry points gain parameters): it is built again, or refused.
        if not (build_if_missing and _build.can_build()):
            raise KernelError(f"{_build.LIB_PATH} was built from other sources than those in {_build.SRC_DIR} "
                              "and cannot be rebuilt here; run __graft_entry__.build()")
        print(f"[bc4g] {_build.LIB_PATH} was built from other sources than those beside it: building it again",
              file=sys.stderr, flush=True)
        _build.build(verbose=True)
    # PyTorch first: it brings a HIP runtime of its own, and the library must bind to that one.  Loaded
    # before torch, the library pulls in the system's runtime instead, the process then holds two, and
    # the library's launches fail ("no ROCm-capable device is detected").
    import torch  # noqa: F401
    try:
        lib = ctypes.CDLL(_build.LIB_PATH)
    except OSError as e:
        raise KernelError(f"cannot load {_build.LIB_PATH}: {e}") from None
    lib.bc4g_sources_digest.restype = c_char_p
    lib.bc4g_sources_digest.argtypes = []
    if (lib.bc4g_sources_digest() or b"").decode("ascii", "replace") != _build.sources_digest():
        raise KernelError(f"{_build.LIB_PATH} does not carry the digest of the sources beside it")
    lib.bc4g_last_error.restype = c_char_p
    lib.bc4g_last_error.argtypes = []
    lib.bc4g_version.restype = c_int
    for name, args in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"{_build.LIB_PATH} lacks {name}; rebuild it with "
                              "__graft_entry__.build()") from None
        fn.argtypes = args
        fn.restype = c_int
    _lib = lib
    return lib


_entry: dict = {}
_profiler = profiler()


def call(name: str, *args, cost=None, launches: bool = True) -> None:
    """Calls an entry point of the library.  ``cost``: a function that gives (floating-point
    operations, bytes to move at least) of this call, asked only while the profiler is on.
    ``launches`` False: a question to the library that starts no kernel (the profiler leaves it out)."""
    fn = _entry.get(name)
    if fn is None:
        fn = _entry[name] = getattr(load(), name)
    if _profiler.enabled and launches:
        mark = _profiler.begin(name[5:] if name.startswith("bc4g_") else name, cost)
        status = fn(*args)
        _profiler.end(mark)
    else:
        status = fn(*args)
    if status != 0:
        raise KernelError(load().bc4g_last_error().decode("utf-8", "replace"))
