"""The host core: the C++ module that keeps the cache pages, schedules, packs steps and
launches a step's kernels.  This file only finds (or builds) and loads it.

There is no Python stand-in: when the module cannot be built or loaded, importing anything
that needs it raises.
"""

from __future__ import annotations

import importlib.util
import sys

from .kernels import build

MODULE_NAME = "mercury_host"


class HostCoreError(RuntimeError):
    pass


def _load():
    try:
        path = build.build_library(build.HOST_NAME, force=False)
    except build.BuildError as e:
        raise HostCoreError(f"the host core is not built and could not be built: {e}") from e
    spec = importlib.util.spec_from_file_location(MODULE_NAME, str(path))
    if spec is None or spec.loader is None:
        raise HostCoreError(f"cannot load {path}")
    module = importlib.util.module_from_spec(spec)
    try:
        spec.loader.exec_module(module)
    except ImportError as e:
        raise HostCoreError(f"cannot load {path}: {e}") from e
    sys.modules[MODULE_NAME] = module
    return module


core = sys.modules.get(MODULE_NAME) or _load()
