"""Builds the HIP libraries for gfx950 with hipcc and finds built ones.

Two kinds of library: ``core`` (embedding, norm, rotary + cache write, matrix
products, sampling) and ``attn_d<D>`` (attention for head size D; one per head
size that a model needs); beside them ``measure`` (stream and matrix-instruction loops for
the benchmark's measured peaks) and the plain C++ references of the same operations,
built with the host compiler for the tests.  A library's file name carries a hash of its sources
and flags, so a library built from other sources is never loaded.  Libraries are
kept in ``kernels/lib`` inside the package, or, if that folder cannot be written,
in a per-user folder under the system's temporary directory (or
``$LLMLAB_BUILD_DIR``).
"""
from __future__ import annotations

import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, List, Optional, Sequence

ARCH = "gfx950"
CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
CORE_SOURCES = ("elementwise.hip", "gemm.hip", "decode.hip", "sampling.hip")
ATTENTION_SOURCE = "attention.hip"
HEADERS = ("common.h",)
CORE_HEADERS = ("no_alloc.h",)      # included by the core sources only
FLAGS = ("-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")
DEFAULT_HEAD_DIMS = (16, 32, 64, 128)


def _say(msg: str) -> None:
    print(f"[llm-inference-lab_amd] {msg}", file=sys.stderr, flush=True)


def _hash(sources: Sequence[str], defines: Sequence[str]) -> str:
    h = hashlib.sha256()
    extra = CORE_HEADERS if tuple(sources) == CORE_SOURCES else ()
    for name in list(sources) + list(HEADERS) + list(extra):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    h.update(" ".join(FLAGS).encode())
    h.update(" ".join(defines).encode())
    return h.hexdigest()[:12]


def _fallback_dir() -> str:
    base = os.environ.get("LLMLAB_BUILD_DIR")
    if base:
        return base
    return os.path.join(tempfile.gettempdir(), f"llmlab_amd_build_{os.getuid()}")


def _search_dirs() -> List[str]:
    return [LIB_DIR, _fallback_dir()]


def _writable_dir() -> str:
    for d in _search_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel libraries; set LLMLAB_BUILD_DIR")


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc not found: the kernels are HIP sources compiled for gfx950")


def _lib_name(kind: str, sources, defines) -> str:
    return f"libllmlab_{kind}.{_hash(sources, defines)}.so"


def _compile(kind: str, sources: Sequence[str], defines: Sequence[str], force: bool) -> str:
    defines = tuple(defines)
    name = _lib_name(kind, sources, defines)
    if not force:
        for d in _search_dirs():
            path = os.path.join(d, name)
            if os.path.isfile(path):
                return path
    out_dir = _writable_dir()
    path = os.path.join(out_dir, name)
    tmp = f"{path}.{os.getpid()}.tmp"
    cmd = [hipcc_path(), *FLAGS, *defines, "-I", CSRC,
           *[os.path.join(CSRC, s) for s in sources], "-o", tmp]
    _say(f"compiling {kind} for {ARCH} ({', '.join(sources)}) ...")
    start = time.time()
    done = threading.Event()

    def heartbeat():
        while not done.wait(10.0):
            _say(f"  still compiling {kind} ({time.time() - start:.0f} s)")
    t = threading.Thread(target=heartbeat, daemon=True)
    t.start()
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    finally:
        done.set()
    if proc.returncode != 0:
        lines = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l]
        raise RuntimeError(f"hipcc failed for {kind}:\n" + "\n".join(lines[-40:]))
    os.replace(tmp, path)
    # older builds of the same library are of no use any more
    for old in glob.glob(os.path.join(out_dir, f"libllmlab_{kind}.*.so")):
        if old != path:
            try:
                os.remove(old)
            except OSError:
                pass
    _say(f"built {os.path.basename(path)} in {time.time() - start:.1f} s")
    return path


def core_library(force: bool = False) -> str:
    return _compile("core", CORE_SOURCES, (), force)


def attention_library(head_dim: int, force: bool = False) -> str:
    if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
        from ..config.errors import UnsupportedSizeError
        raise UnsupportedSizeError(
            f"attention kernels take head sizes that are multiples of 16 from 16 to 256, "
            f"got {head_dim}")
    return _compile(f"attn_d{head_dim}", (ATTENTION_SOURCE,), (f"-DHEAD_DIM={head_dim}",), force)


MEASURE_SOURCE = "measure.hip"


def measure_library(force: bool = False) -> str:
    """Stream and matrix-instruction loops that measure what the machine gives
    (``csrc/measure.hip``).  The benchmark loads it; the product never does."""
    return _compile("measure", (MEASURE_SOURCE,), (), force)


REFERENCE_SOURCE = "reference.cpp"


def reference_library(force: bool = False) -> str:
    """The plain C++ references of the kernels' operations (``csrc/reference.cpp``), built with
    the host compiler.  Tests load it; the product never does."""
    with open(os.path.join(CSRC, REFERENCE_SOURCE), "rb") as f:
        digest = hashlib.sha256(f.read()).hexdigest()[:12]
    name = f"libllmlab_reference.{digest}.so"
    if not force:
        for d in _search_dirs():
            if os.path.isfile(os.path.join(d, name)):
                return os.path.join(d, name)
    compiler = next((c for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"),
                                 shutil.which("clang++")) if c), None)
    if compiler is None:
        raise RuntimeError("no host C++ compiler found for the plain references")
    out_dir = _writable_dir()
    path = os.path.join(out_dir, name)
    tmp = f"{path}.{os.getpid()}.tmp"
    proc = subprocess.run([compiler, "-O2", "-std=c++17", "-fPIC", "-shared",
                           os.path.join(CSRC, REFERENCE_SOURCE), "-o", tmp],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("the host compiler failed for the plain references:\n" + proc.stdout[-4000:])
    os.replace(tmp, path)
    for old in glob.glob(os.path.join(out_dir, "libllmlab_reference.*.so")):
        if old != path:
            try:
                os.remove(old)
            except OSError:
                pass
    _say(f"built {name}")
    return path


def library(kind: str, parameter=None, force: bool = False) -> str:
    """The library a part names in ``kernel_libraries()``: ``("core", None)`` or
    ``("attention", head_dim)``."""
    if kind == "core":
        return core_library(force)
    if kind == "attention":
        return attention_library(int(parameter), force)
    raise ValueError(f"no kernel library of kind '{kind}'")


def build_all(head_dims: Sequence[int] = DEFAULT_HEAD_DIMS, force: bool = True) -> Dict[str, str]:
    """Compile the core library and the attention libraries of the given head sizes."""
    out = {"core": core_library(force)}
    for d in head_dims:
        out[f"attn_d{d}"] = attention_library(d, force)
    out["measure"] = measure_library(force)
    out["reference"] = reference_library(force)
    return out
