"""Compile and load the HIP kernels (gfx950 only).

Each source under ``csrc/`` becomes one shared library with C entry points, built
by ``hipcc`` and loaded with ``ctypes``. The attention file is compiled once per
head size (``-DSOC_HEAD_DIM``), so a model compiles what its configuration
needs. A library's file name carries a hash of its sources and flags: a stale
build is never loaded. Libraries live in ``csrc/_build`` inside the package, or
in a per-user folder under the temp directory if the package is read-only.

The reference builds one CUDA extension ahead of time (model/kernels/setup.py:1-41)
and fails fast if it is absent (model/kernels/__init__.py:82-92); here a missing
library is compiled at first use, and a failed compile is an error, never a
fallback.
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
# Packed float32 instructions are kept off: some of their forms have returned wrong
# results on this hardware generation.
HIPCC_FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-fno-gpu-rdc", "-Wno-unused-value"]
# Attention up to head size 128: MFMA accumulators stay in ordinary vector registers. The
# softmax rescales them with vector instructions, and copies to and from the accumulation
# registers would cost more than the products. Larger heads need both register files.
MFMA_VGPR_FLAGS = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
MFMA_VGPR_MAX_HEAD = 128

SOURCES = {"elementwise": "elementwise.hip", "gemm": "gemm.hip", "sampling": "sampling.hip",
           "attention": "attention.hip"}
# head sizes built ahead by build_all(): the common ones and those the tests use, so that
# no test compiles on the GPU box
COMMON_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 256)

_loaded = {}
_lock = threading.Lock()
_dir_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                           "the HIP kernels cannot be built and there is no other path")


_build_dir_cache = None


def _build_dir() -> Path:
    global _build_dir_cache
    with _dir_lock:
        if _build_dir_cache is None:
            inside = CSRC / "_build"
            try:
                inside.mkdir(exist_ok=True)
                probe = inside / f".probe{os.getpid()}"
                probe.write_text("")
                probe.unlink()
                _build_dir_cache = inside
            except OSError:
                d = Path(tempfile.gettempdir()) / f"socrates_amd_build_{os.getuid()}"
                d.mkdir(parents=True, exist_ok=True)
                _build_dir_cache = d
        return _build_dir_cache


def _variant(name: str, head_dim=None):
    if name == "attention":
        if head_dim is None:
            raise ValueError("the attention library is built per head size")
        extra = MFMA_VGPR_FLAGS if head_dim <= MFMA_VGPR_MAX_HEAD else []
        return f"attention_d{head_dim}", [f"-DSOC_HEAD_DIM={head_dim}"] + extra
    return name, []


def _digest(name: str, defines) -> str:
    h = hashlib.sha256()
    h.update((CSRC / SOURCES[name]).read_bytes())
    for header in sorted(CSRC.glob("*.h")):
        h.update(header.read_bytes())
    h.update(" ".join(HIPCC_FLAGS + list(defines)).encode())
    return h.hexdigest()[:12]


def library_path(name: str, head_dim=None, folder: Path = None) -> Path:
    tag, defines = _variant(name, head_dim)
    return (folder or _build_dir()) / f"libsoc_{tag}.{_digest(name, defines)}.so"


def compile_library(name: str, head_dim=None, force=False, quiet=False) -> Path:
    """Compile one library if its current build is absent (or ``force``). Returns its path."""
    tag, defines = _variant(name, head_dim)
    out = library_path(name, head_dim)
    if out.exists() and not force:
        return out
    for old in out.parent.glob(f"libsoc_{tag}.*.so"):
        try:
            old.unlink()
        except OSError:
            pass
    tmp = out.with_suffix(f".tmp{os.getpid()}.so")
    cmd = [_hipcc()] + HIPCC_FLAGS + defines + [str(CSRC / SOURCES[name]), "-o", str(tmp)]
    if not quiet:
        print(f"[socrates_amd] compiling {tag} for {ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                            cwd=str(out.parent))
    # a line now and then while the compiler works
    while True:
        try:
            output, _ = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if not quiet:
                print(f"[socrates_amd] still compiling {tag} ({time.time() - t0:.0f} s)",
                      file=sys.stderr, flush=True)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed for {tag}:\n{' '.join(cmd)}\n{output}")
    os.replace(tmp, out)
    if not quiet:
        print(f"[socrates_amd] built {out.name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def load_library(name: str, head_dim=None) -> ctypes.CDLL:
    """The loaded library, compiled first if needed. Raises KernelBuildError if it cannot be
    built or loaded; there is no fallback."""
    key = (name, head_dim)
    with _lock:
        lib = _loaded.get(key)
        if lib is None:
            path = compile_library(name, head_dim)
            try:
                lib = ctypes.CDLL(str(path))
            except OSError as e:
                raise KernelBuildError(f"cannot load {path}: {e}") from e
            _loaded[key] = lib
        return lib


def build_all(head_dims=COMMON_HEAD_DIMS, force=True, jobs=None) -> list:
    """Compile every library (the attention file for each of ``head_dims``)."""
    from concurrent.futures import ThreadPoolExecutor
    tasks = [(n, None) for n in SOURCES if n != "attention"] + [("attention", d) for d in head_dims]
    jobs = jobs or min(len(tasks), max(1, (os.cpu_count() or 2) // 2), 8)
    with ThreadPoolExecutor(jobs) as pool:
        return list(pool.map(lambda t: compile_library(t[0], t[1], force=force), tasks))
