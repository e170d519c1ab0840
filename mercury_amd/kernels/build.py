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
        "attention_out.hip",
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


# The host core: C++ (pybind11) for the cache manager, the scheduler, step packing, the walk
# over a step's program and the built-in operations' launch sequences.  Compiled with the host compiler; it reaches the kernel libraries
# and the HIP runtime through dlopen/dlsym, so it links against neither.
HOST_NAME = "host"
HOST_DIR = CSRC / "host"     # what knows no operation: cache, scheduler, packer, program walk
OPS_DIR = CSRC / "ops"       # the built-in operations, their launch sequences and choices
KERNEL_HEADER = CSRC / "mercury_kernels.h"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off", "-pthread",
              "-D__HIP_PLATFORM_AMD__", "-Wall", "-Wno-unused-function"]


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
    return "mercury_host.so" if name == HOST_NAME else f"libmercury_{name}.so"


def _sources(name: str) -> list:
    if name == HOST_NAME:
        return sorted(HOST_DIR.glob("*.cc")) + sorted(OPS_DIR.glob("*.cc"))
    return [CSRC / s for s in LIBRARIES[name]]


def _host_headers() -> list:
    return sorted(HOST_DIR.glob("*.h")) + sorted(OPS_DIR.glob("*.h"))


def kernel_prototypes() -> dict:
    """library name -> [(function name, return type, [parameter types])], read from the one
    declaration of the kernel libraries' C interface (``csrc/mercury_kernels.h``).  A line
    ``// @library NAME`` says which library the declarations after it belong to; what stands
    before the first such line is in every library."""
    import re

    out = {name: [] for name in LIBRARIES}
    current = None
    text = KERNEL_HEADER.read_text()
    # keep the markers, drop every other comment
    text = re.sub(r"//\s*@library\s+(\w+).*", r"@library \1;", text)
    text = re.sub(r"//.*", "", text)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for statement in text.split(";"):
        statement = " ".join(statement.split())
        marker = re.search(r"@library (\w+)$", statement)
        if marker:
            current = marker.group(1)
            if current not in out:
                raise BuildError(f"{KERNEL_HEADER.name} names an unknown library {current!r}")
            continue
        match = re.search(r"([\w ]+?[\w\*]) ?\b(mk_\w+) ?\((.*)\)$", statement)
        if not match:
            continue
        returns, name, params = match.group(1).strip(), match.group(2), match.group(3).strip()
        returns = returns.split("{")[-1].strip()          # the extern "C" brace
        types = []
        if params and params != "void":
            for param in params.split(","):
                param = param.strip()
                types.append("pointer" if "*" in param else " ".join(param.split()[:-1]))
        for lib in ([current] if current else list(out)):
            out[lib].append((name, returns, types))
    return out


def kernel_abi_version() -> int:
    """MK_ABI_VERSION as the header defines it."""
    import re

    match = re.search(r"#define\s+MK_ABI_VERSION\s+(\d+)", KERNEL_HEADER.read_text())
    if not match:
        raise BuildError(f"{KERNEL_HEADER.name} defines no MK_ABI_VERSION")
    return int(match.group(1))


def _write_kernel_names(folder: Path) -> Path:
    """The lists of entry points by library as X-macros, for the host core's table of function
    pointers (their types come from the declarations themselves, by decltype)."""
    common = {"mk_last_error", "mk_abi_version"}
    lines = ["// Written by the build from mercury_kernels.h; not a source file."]
    for lib, protos in kernel_prototypes().items():
        names = " ".join(f"X({name})" for name, _, _ in protos if name not in common)
        lines.append(f"#define MK_{lib.upper()}_FUNCTIONS(X) {names}")
    folder.mkdir(parents=True, exist_ok=True)
    path = folder / "kernel_names.inc"
    text = "\n".join(lines) + "\n"
    if not path.is_file() or path.read_text() != text:
        path.write_text(text)
    return path


def source_hash(name: str) -> str:
    digest = hashlib.sha256()
    headers = sorted(CSRC.glob("*.h"))
    if name == HOST_NAME:
        digest.update(" ".join(HOST_FLAGS).encode())
        digest.update(sys.version.encode())
        headers += _host_headers()
    else:
        digest.update(" ".join(HIPCC_FLAGS).encode())
    for path in _sources(name) + headers:
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


def _host_compiler() -> str:
    for candidate in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++")):
        if candidate and Path(candidate).exists():
            return candidate
    raise BuildError("no C++ compiler was found for the host core (looked at $CXX, g++, c++)")


def _rocm_root() -> Path:
    for candidate in (os.environ.get("ROCM_PATH"), "/opt/rocm"):
        if candidate and (Path(candidate) / "include" / "hip").is_dir():
            return Path(candidate)
    raise BuildError("the ROCm headers were not found (looked at $ROCM_PATH and /opt/rocm)")


def _host_commands(sources: list, objects: list, target: Path, generated: Path) -> tuple:
    import sysconfig

    import pybind11

    cxx, rocm = _host_compiler(), _rocm_root()
    includes = ["-I", pybind11.get_include(), "-I", sysconfig.get_paths()["include"],
                "-I", str(rocm / "include"), "-I", str(CSRC), "-I", str(generated)]
    compiles = [[cxx, *HOST_FLAGS, *includes, "-c", str(src), "-o", str(obj)]
                for src, obj in zip(sources, objects)]
    # No HIP runtime is linked: the core finds, at run time, the one the process already uses.
    link = [cxx, "-shared", "-pthread", "-o", str(target), *map(str, objects), "-ldl"]
    return compiles, link


def build_library(name: str, force: bool = False, verbose: bool = True) -> Path:
    """Compile one library (a kernel library, or the host core "host") and return its path."""
    if name != HOST_NAME and name not in LIBRARIES:
        raise BuildError(f"unknown kernel library {name!r}; known: {sorted(LIBRARIES)}")
    if not force:
        found = find_library(name)
        if found is not None:
            return found
    out_dir = next((d for d in library_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the kernel library")
    obj_dir = out_dir / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    sources = _sources(name)
    objects = [obj_dir / f"{name}-{src.stem}.o" for src in sources]
    target = out_dir / library_name(name)
    partial = out_dir / (library_name(name) + f".{os.getpid()}.tmp")
    if name == HOST_NAME:
        if verbose:
            _say(f"compiling the host core: {len(sources)} sources -> {out_dir}")
        generated = obj_dir / "include"
        _write_kernel_names(generated)
        compiles, link = _host_commands(sources, objects, partial, generated)
    else:
        hipcc = _hipcc()
        if verbose:
            _say(f"compiling kernel library '{name}' for {ARCH}: {len(sources)} sources -> {out_dir}")
        compiles = [[hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
                    for src, obj in zip(sources, objects)]
        link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o",
                str(partial), *map(str, objects)]
    threads, errors = [], []
    headers = b"".join(p.read_bytes() for p in sorted(CSRC.glob("*.h")) + _host_headers())
    for src, obj, cmd in zip(sources, objects, compiles):
        # An object whose command, source and headers are what they were is kept, unless the
        # caller asked for everything to be compiled again.
        wanted = hashlib.sha256(" ".join(cmd).encode() + src.read_bytes() + headers).hexdigest()
        mark = obj.with_suffix(".o.stamp")
        if not force and obj.is_file() and mark.is_file() and mark.read_text().strip() == wanted:
            continue

        def work(cmd=cmd, src=src, mark=mark, wanted=wanted):
            try:
                _run_with_heartbeat(cmd, src.name)
                mark.write_text(wanted + "\n")
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
    _run_with_heartbeat(link, library_name(name))
    os.replace(partial, target)
    _stamp(target).write_text(source_hash(name) + "\n")
    if verbose:
        _say(f"built {target}")
    return target


def build_all(force: bool = True, verbose: bool = True) -> dict:
    return {name: build_library(name, force=force, verbose=verbose)
            for name in [*LIBRARIES, HOST_NAME]}


if __name__ == "__main__":
    for lib_name, lib_path in build_all(force="--no-force" not in sys.argv).items():
        print(lib_name, lib_path)
