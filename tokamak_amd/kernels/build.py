"""Compile the HIP sources for gfx950 and load them through ctypes.

Each ``csrc/<name>.hip`` becomes ``csrc/libtk_<name>.so`` beside it.  A library
is loaded when first used; if it is missing or older than its sources it is
compiled then (in the source tree when that is writable, otherwise under a
per-user folder in the temporary directory), printing a line when it starts and
about every ten seconds while it runs.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
# packed float32 instructions are switched off for every kernel of this engine
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
LIBRARIES = ("elementwise", "gemm_tiled", "attention_generic", "sampling", "gemm_mfma",
             "gemm_wholek", "attention_mfma", "blas_lt", "peaks", "replay")
# libraries a source links against (blas_lt is host code around hipBLASLt)
LINK_FLAGS = {"blas_lt": ["-lhipblaslt"]}

_loaded: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def sources_of(name: str) -> list[Path]:
    """The library's source and the headers of this folder that it includes (directly
    or through another of them)."""
    src = CSRC / f"{name}.hip"
    if not src.is_file():
        raise KernelBuildError(f"no kernel source {src}")
    found, todo = [src], [src]
    while todo:
        for line in todo.pop().read_text().splitlines():
            line = line.strip()
            if line.startswith("#include \""):
                header = CSRC / line.split('"')[1]
                if header.is_file() and header not in found:
                    found.append(header)
                    todo.append(header)
    return [src, *sorted(found[1:])]


def _digest(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join([*HIPCC_FLAGS, *LINK_FLAGS.get(name, [])]).encode())
    for path in sources_of(name):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()


def _hipcc() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).is_file():
            return cand
    return None


def _fallback_dir() -> Path:
    d = Path(tempfile.gettempdir()) / f"tokamak_amd-{os.getuid()}"
    d.mkdir(parents=True, exist_ok=True)
    return d


def _candidates(name: str) -> list[Path]:
    return [CSRC / f"libtk_{name}.so", _fallback_dir() / f"libtk_{name}.so"]


def _is_current(lib: Path, digest: str) -> bool:
    stamp = lib.with_suffix(".so.stamp")
    return lib.is_file() and stamp.is_file() and stamp.read_text().strip() == digest


def compile_library(name: str, *, quiet: bool = False) -> Path:
    """Compile one library now, whatever is there; return its path."""
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelBuildError("hipcc not found: cannot compile the HIP kernels")
    digest = _digest(name)
    out_dir = CSRC if os.access(CSRC, os.W_OK) else _fallback_dir()
    lib = out_dir / f"libtk_{name}.so"
    tmp = out_dir / f".libtk_{name}.{os.getpid()}.so"
    cmd = [hipcc, *HIPCC_FLAGS, f"-I{CSRC}", str(CSRC / f"{name}.hip"), "-o", str(tmp),
           *LINK_FLAGS.get(name, [])]
    if not quiet:
        print(f"[tokamak_amd] compiling {name}.hip for {ARCH} ...", file=sys.stderr, flush=True)
    start = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    while True:
        try:
            output, _ = proc.communicate(timeout=10)
            break
        except subprocess.TimeoutExpired:
            if not quiet:
                print(f"[tokamak_amd] still compiling {name}.hip ({time.time() - start:.0f} s)",
                      file=sys.stderr, flush=True)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed for {name}.hip:\n{output}")
    os.replace(tmp, lib)
    lib.with_suffix(".so.stamp").write_text(digest + "\n")
    if not quiet:
        print(f"[tokamak_amd] built {lib.name} in {time.time() - start:.0f} s", file=sys.stderr,
              flush=True)
    return lib


def available_libraries() -> list[str]:
    return [n for n in LIBRARIES if (CSRC / f"{n}.hip").is_file()]


def build_all(*, force: bool = True, jobs: int = 4) -> list[Path]:
    """Compile every library (``force``: also those that are current)."""
    from concurrent.futures import ThreadPoolExecutor

    names = available_libraries()
    todo = [n for n in names if force or not any(_is_current(c, _digest(n)) for c in _candidates(n))]
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        return list(pool.map(compile_library, todo))


def load_library(name: str) -> ctypes.CDLL:
    """The loaded library ``name``; compiled first if missing or stale."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        digest = _digest(name)
        path = next((c for c in _candidates(name) if _is_current(c, digest)), None)
        if path is None:
            stale = next((c for c in _candidates(name) if c.is_file()), None)
            if _hipcc() is not None:
                path = compile_library(name)
            elif stale is not None:
                raise KernelBuildError(
                    f"{stale} is older than its sources and hipcc is not available to rebuild it")
            else:
                raise KernelBuildError(
                    f"kernel library libtk_{name}.so is not built and hipcc is not available")
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as err:
            raise KernelBuildError(f"cannot load {path}: {err}") from err
        _loaded[name] = lib
        return lib
