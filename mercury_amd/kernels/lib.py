"""Load the kernel libraries through ctypes and declare their C signatures.

There is no fallback: when a library cannot be built or loaded, :func:`load` raises, and so
does every op that would have called into it.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_ulonglong, c_void_p

from . import build

ABI_VERSION = 12

P, I, F, L = c_void_p, c_int, c_float, c_longlong

# name -> argument types (every function returns int)
_SIGNATURES = {
    "core": {
        "mk_embed": [P, P, I, P, I, I, I, P],
        "mk_rmsnorm": [P, P, I, L, P, I, F, P, P, I, I, I, P],
        "mk_silu_mul": [P, P, I, I, I, P],
        "mk_rope_kv_write": [P, I, I, P, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, I, P],
        "mk_linear_generic": [P, P, I, P, I, P, I, I, I, I, I, I, I, P],
        "mk_attention_generic": [P, I, P, I, P, P, I, P, P, P, I, I, I, I, I, F, I, I, P],
        "mk_qkv_finish": [P, I, L, P, I, P, I, P, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, P],
        "mk_argmax": [P, I, I, L, P, P, P],
        "mk_argmax_static_max_rows": [],
        "mk_argmax_static": [P, I, I, L, P, P],
        "mk_sample_scratch_bytes": [I, I],
        "mk_sample": [P, I, I, L, P, P, P, P, P, P],
        "mk_fill_normal": [P, I, L, c_ulonglong, F, F, P],
    },
    "mfma": {
        "mk_linear_skinny_slices": [I, I, I],
        "mk_linear_skinny": [P, P, P, I, I, I, I, P],
        "mk_linear_skinny_unsplit": [I, I, I],
        "mk_linear_skinny_acc": [P, P, P, I, P, I, I, I, P],
        "mk_gated_skinny": [P, P, P, I, I, I, P],
        "mk_qkv_skinny": [P, P, P, I, P, P, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, P],
        "mk_qkv_tiled": [P, P, P, I, P, P, P, I, P, P, P, I, P, P, I, I, I, I, I, I, I, I, P],
        "mk_gated_tiled_config": [I, I, I],
        "mk_gated_tiled": [P, P, P, I, I, I, I, P],
        "mk_linear_tiled_slices": [I, I, I],
        "mk_linear_tiled_partials": [P, P, P, I, I, I, I, P],
        "mk_linear_tiled_configs": [],
        "mk_linear_tiled_config": [I, I, I, I],
        "mk_linear_tiled": [P, P, P, I, P, I, I, I, I, I, I, I, P],
        "mk_attention_mfma_supported": [I, I],
        "mk_attention_mfma_max_rows": [I],
        "mk_attention_mfma_staged": [I, I],
        "mk_attention_mfma_wide": [I],
        "mk_attention_mfma": [P, I, P, I, P, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, I, I, I, P, P, P],
    },
}

_RETURNS_SIZE = {"mk_sample_scratch_bytes"}    # byte counts; everything else returns int

_loaded: dict = {}


class KernelLibraryError(RuntimeError):
    pass


def load(name: str = "core") -> ctypes.CDLL:
    """The library `name`, built first if no current build exists."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    try:
        path = build.build_library(name, force=False)
    except build.BuildError as e:
        raise KernelLibraryError(
            f"the gfx950 kernel library '{name}' is not built and could not be built: {e}"
        ) from e
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from e
    lib.mk_last_error.restype = c_char_p
    lib.mk_last_error.argtypes = []
    lib.mk_abi_version.restype = c_int
    if lib.mk_abi_version() != ABI_VERSION:
        raise KernelLibraryError(
            f"{path} has ABI {lib.mk_abi_version()}, this package expects {ABI_VERSION}; rebuild"
        )
    for fn_name, argtypes in _SIGNATURES[name].items():
        fn = getattr(lib, fn_name)
        fn.argtypes = argtypes
        fn.restype = c_longlong if fn_name in _RETURNS_SIZE else c_int
    # The host core launches a step's kernels itself and decides which kernel runs what: it
    # opens the same library.
    from ..hostcore import core

    core.load_kernels(name, str(path))
    _loaded[name] = lib
    return lib


def check(lib: ctypes.CDLL, code: int, what: str) -> None:
    if code != 0:
        message = lib.mk_last_error().decode(errors="replace")
        raise KernelLibraryError(f"{what}: {message}")
