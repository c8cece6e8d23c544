"""Loads the gfx950 kernel library and declares its entry points for ctypes.

There is no fallback: when the library cannot be built or loaded, or no GPU is
present when a kernel is called, the caller gets an error.  torch must be
imported before the library so that both use the same HIP runtime.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_size_t, c_uint32, c_void_p

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

from tokasaurus_amd.kernels import build as _build

ABI_VERSION = 9


class KernelError(RuntimeError):
    """A kernel refused its arguments, or its launch failed."""


_P = c_void_p
_SIGNATURES: dict[str, list] = {
    "tk_embed_gather": [c_int, _P, _P, _P, _P, c_int, c_int, c_int, _P],
    "tk_rmsnorm": [c_int, _P, _P, c_int, _P, c_int, c_int, c_float, _P],
    "tk_swiglu": [c_int, _P, _P, c_int, c_int, _P],
    "tk_gather_rows": [c_int, _P, c_int, _P, _P, c_int, c_int, _P],
    "tk_rope_table": [_P, _P, _P, c_int, c_int, _P],
    "tk_rope_append": [c_int, _P, c_int, _P, _P, _P, c_int, _P, _P, _P, _P]
    + [c_int] * 6
    + [_P],
    "tk_fill_u32": [_P, c_uint32, c_size_t, _P],
    "tk_gemm_generic": [c_int, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, _P],
    "tk_paged_attention_generic": [c_int, _P, c_int, _P, c_int, _P, _P, _P, c_int, _P, _P]
    + [c_int] * 6
    + [c_float, _P],
    "tk_paged_attention_mfma": [_P, c_int, _P, c_int, _P, _P, _P, c_int, _P, _P, _P, _P]
    + [c_int] * 7
    + [c_float, c_int, c_int, c_int, _P, _P, _P],
    "tk_gemm_skinny_bf16": [_P, c_int, _P, _P, c_int, _P, c_int, _P, c_int, c_float]
    + [c_int] * 8
    + [_P],
    "tk_add": [c_int, _P, _P, _P, c_size_t, _P],
    "tk_sample": [_P, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "tk_sample_chunks": [c_int],
}

_lib: ctypes.CDLL | None = None


def load() -> ctypes.CDLL:
    """The loaded library; builds it first when it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    path = _build.ensure_built()
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelError(f"cannot load the kernel library {path}: {e}") from None
    lib.tk_last_error.restype = c_char_p
    lib.tk_last_error.argtypes = []
    lib.tk_abi_version.restype = c_int
    if lib.tk_abi_version() != ABI_VERSION:
        raise KernelError(
            f"kernel library {path} has ABI {lib.tk_abi_version()}, expected {ABI_VERSION}; "
            "rebuild it with `python -m tokasaurus_amd.kernels.build`"
        )
    for name, argtypes in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"kernel library {path} lacks entry point {name}") from None
        fn.argtypes = argtypes
        fn.restype = c_int
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    """Call an entry point and raise KernelError with its message on refusal."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(lib.tk_last_error().decode(errors="replace"))
