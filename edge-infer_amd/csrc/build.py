"""Compiles the HIP sources of this folder for gfx950, one shared library each.

A library is compiled the first time something needs it (a line is printed when a
compilation starts and every twenty seconds while it runs) and reused afterwards:
a stamp beside it records the hash of its source, the shared header and the
flags.  `build_all()` compiles every library, whatever is already there.
"""
from __future__ import annotations

import functools
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

SOURCE_DIR = Path(__file__).resolve().parent
LIBRARIES = ("rowwise", "rope_store", "attention_generic", "attention_mfma", "gemm_f32",
             "gemm_bf16", "sampling", "peaks")
ARCH = "gfx950"
# packed-fp32 instructions are switched off for every device compilation
FLAGS = ("-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option")


class BuildError(RuntimeError):
    pass


def available_libraries():
    return tuple(name for name in LIBRARIES if (SOURCE_DIR / f"{name}.hip").is_file())


@functools.lru_cache(maxsize=1)
def _build_dir() -> Path:
    override = os.environ.get("EDGE_INFER_BUILD_DIR")
    candidates = [Path(override)] if override else []
    candidates.append(SOURCE_DIR / "_build")
    candidates.append(Path(tempfile.gettempdir()) / f"edge_infer_amd_build_{os.getuid()}")
    for directory in candidates:
        try:
            directory.mkdir(parents=True, exist_ok=True)
            probe = directory / f".probe_{os.getpid()}"
            probe.write_text("")
            probe.unlink()
            return directory
        except OSError:
            continue
    raise BuildError("no writable folder for compiled kernels; set EDGE_INFER_BUILD_DIR")


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).is_file():
            return candidate
    raise BuildError("hipcc was not found: the HIP kernels cannot be compiled, and there is "
                     "no other implementation to fall back to")


def _stamp(name: str) -> str:
    digest = hashlib.sha256()
    digest.update((SOURCE_DIR / f"{name}.hip").read_bytes())
    for header in sorted(SOURCE_DIR.glob("*.h")):
        digest.update(header.read_bytes())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()


def library_path(name: str) -> Path:
    """Path of the built library, looking in the in-tree folder first."""
    in_tree = SOURCE_DIR / "_build" / f"libei_{name}.so"
    if in_tree.is_file():
        return in_tree
    return _build_dir() / f"libei_{name}.so"


def is_current(name: str) -> bool:
    path = library_path(name)
    stamp = path.with_suffix(".stamp")
    return path.is_file() and stamp.is_file() and stamp.read_text().strip() == _stamp(name)


def build_library(name: str, force: bool = False, quiet: bool = False) -> Path:
    if name not in available_libraries():
        raise BuildError(f"unknown kernel library '{name}'")
    if not force and is_current(name):
        return library_path(name)
    directory = _build_dir()
    target = directory / f"libei_{name}.so"
    partial = directory / f"libei_{name}.{os.getpid()}.tmp.so"
    command = [_hipcc(), *FLAGS, str(SOURCE_DIR / f"{name}.hip"), "-o", str(partial)]
    if not quiet:
        print(f"[edge-infer] compiling {name}.hip for {ARCH} ...", file=sys.stderr, flush=True)
    started = time.time()
    process = subprocess.Popen(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                               text=True, cwd=str(directory))
    last = started
    while True:
        try:
            output, _ = process.communicate(timeout=5)
            break
        except subprocess.TimeoutExpired:
            if not quiet and time.time() - last >= 20:
                last = time.time()
                print(f"[edge-infer] still compiling {name}.hip "
                      f"({int(last - started)} s)", file=sys.stderr, flush=True)
    if process.returncode != 0:
        partial.unlink(missing_ok=True)
        raise BuildError(f"hipcc failed for {name}.hip:\n{output}")
    os.replace(partial, target)
    target.with_suffix(".stamp").write_text(_stamp(name) + "\n")
    if not quiet:
        print(f"[edge-infer] compiled {name}.hip in {time.time() - started:.0f} s",
              file=sys.stderr, flush=True)
    return target


def build_libraries(names, force: bool = False, jobs: int = 8) -> None:
    """Compile those of `names` that are not built yet (all of them with `force`), side by
    side: what a model needs is then ready after the longest compilation, not their sum."""
    names = [name for name in dict.fromkeys(names) if force or not is_current(name)]
    if not names:
        return
    _build_dir()
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(names)))) as pool:
        for _ in pool.map(lambda n: build_library(n, force=force), names):
            pass


def build_all(force: bool = True, jobs: int = 8) -> None:
    build_libraries(available_libraries(), force=force, jobs=jobs)
