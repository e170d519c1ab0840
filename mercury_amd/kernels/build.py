"""Compile the HIP sources under ``mercury_amd/csrc`` for gfx950 into shared libraries.

The sources are grouped into libraries so that a run compiles only what it needs: ``core``
holds the float32-arithmetic kernels every model and dtype uses, ``mfma`` the bfloat16
matrix-core kernels that only bfloat16 serving loads.  Libraries are written next to the
sources' package (``mercury_amd/lib``); when that folder cannot be written the build goes to
a per-user folder under the system temporary directory.  Beside each library lies a stamp
with the hash of its sources, headers and compiler flags; a library whose stamp does not
match is rebuilt, as is any library when ``force`` is set.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path

ARCH = "gfx950"
PACKAGE_DIR = Path(__file__).resolve().parent.parent
CSRC = PACKAGE_DIR / "csrc"

LIBRARIES = {
    "core": [
        "host_support.hip",
        "elementwise.hip",
        "gemm_generic.hip",
        "attention_generic.hip",
        "sampling.hip",
        "random_fill.hip",
    ],
    "mfma": [
        "host_support.hip",
        "attention_mfma.hip",
        "gemm_mfma.hip",
    ],
}

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # The packed float32 instructions are kept out of generated code on purpose.
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def library_dirs() -> list:
    """Where a built library may live, in search order."""
    dirs = [PACKAGE_DIR / "lib"]
    env = os.environ.get("MERCURY_AMD_BUILD_DIR")
    if env:
        dirs.insert(0, Path(env))
    dirs.append(Path(tempfile.gettempdir()) / f"mercury_amd-{os.getuid()}" / "lib")
    return dirs


def library_name(name: str) -> str:
    return f"libmercury_{name}.so"


def _sources(name: str) -> list:
    return [CSRC / s for s in LIBRARIES[name]]


def source_hash(name: str) -> str:
    digest = hashlib.sha256()
    digest.update(" ".join(HIPCC_FLAGS).encode())
    for path in _sources(name) + sorted(CSRC.glob("*.h")):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()


def _stamp(path: Path) -> Path:
    return path.with_suffix(".stamp")


def find_library(name: str, allow_stale: bool = False) -> Path | None:
    wanted = None
    for folder in library_dirs():
        path = folder / library_name(name)
        if not path.is_file():
            continue
        if allow_stale:
            return path
        wanted = wanted or source_hash(name)
        stamp = _stamp(path)
        if stamp.is_file() and stamp.read_text().strip() == wanted:
            return path
    return None


def _say(message: str) -> None:
    print(f"[mercury_amd] {message}", file=sys.stderr, flush=True)


def _run_with_heartbeat(cmd: list, what: str) -> None:
    """Run a compiler command, printing a line every ten seconds while it works."""
    started = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def beat():
        while not done.wait(10.0):
            _say(f"still compiling {what} ({time.time() - started:.0f} s)")

    thread = threading.Thread(target=beat, daemon=True)
    thread.start()
    output, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{output}")


def build_library(name: str, force: bool = False, verbose: bool = True) -> Path:
    """Compile one library and return its path."""
    if name not in LIBRARIES:
        raise BuildError(f"unknown kernel library {name!r}; known: {sorted(LIBRARIES)}")
    if not force:
        found = find_library(name)
        if found is not None:
            return found
    out_dir = next((d for d in library_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the kernel library")
    hipcc = _hipcc()
    obj_dir = out_dir / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    sources = _sources(name)
    if verbose:
        _say(f"compiling kernel library '{name}' for {ARCH}: {len(sources)} sources -> {out_dir}")
    objects, threads, errors = [], [], []
    for src in sources:
        obj = obj_dir / f"{name}-{src.stem}.o"
        objects.append(obj)
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]

        def work(cmd=cmd, src=src):
            try:
                _run_with_heartbeat(cmd, src.name)
                if verbose:
                    _say(f"compiled {src.name}")
            except BuildError as e:  # collected and raised on the calling thread
                errors.append(e)

        thread = threading.Thread(target=work)
        thread.start()
        threads.append(thread)
    for thread in threads:
        thread.join()
    if errors:
        raise errors[0]
    target = out_dir / library_name(name)
    partial = out_dir / (library_name(name) + f".{os.getpid()}.tmp")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o",
           str(partial), *map(str, objects)]
    _run_with_heartbeat(cmd, library_name(name))
    os.replace(partial, target)
    _stamp(target).write_text(source_hash(name) + "\n")
    if verbose:
        _say(f"built {target}")
    return target


def build_all(force: bool = True, verbose: bool = True) -> dict:
    return {name: build_library(name, force=force, verbose=verbose) for name in LIBRARIES}


if __name__ == "__main__":
    for lib_name, lib_path in build_all(force="--no-force" not in sys.argv).items():
        print(lib_name, lib_path)
