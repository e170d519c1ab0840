"""Load the kernel libraries through ctypes and declare their C signatures.

There is no fallback: when a library cannot be built or loaded, :func:`load` raises, and so
does every op that would have called into it.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_ulonglong, c_void_p

from . import build

ABI_VERSION = build.kernel_abi_version()

_CTYPES = {"pointer": c_void_p, "int": c_int, "float": c_float, "long long": c_longlong,
           "unsigned long long": c_ulonglong, "hipStream_t": c_void_p, "const char*": c_char_p}


def _signatures(name: str) -> dict:
    """function name -> (return ctype, [argument ctypes]) for the library `name`, from the
    declarations in ``csrc/mercury_kernels.h``: the header is the one place a signature is
    written down."""
    out = {}
    for fn_name, returns, params in build.kernel_prototypes()[name]:
        try:
            out[fn_name] = (_CTYPES[returns], [_CTYPES[p] for p in params])
        except KeyError as e:
            raise KernelLibraryError(
                f"{fn_name}: mercury_kernels.h uses a type this loader does not know: {e}") from None
    return out


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
    lib.mk_abi_version.restype = c_int
    lib.mk_abi_version.argtypes = []
    if lib.mk_abi_version() != ABI_VERSION:
        raise KernelLibraryError(
            f"{path} has ABI {lib.mk_abi_version()}, this package expects {ABI_VERSION}; rebuild"
        )
    for fn_name, (restype, argtypes) in _signatures(name).items():
        try:
            fn = getattr(lib, fn_name)
        except AttributeError:
            raise KernelLibraryError(
                f"{path} has no entry point {fn_name}; rebuild the kernel libraries") from None
        fn.argtypes = argtypes
        fn.restype = restype
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
