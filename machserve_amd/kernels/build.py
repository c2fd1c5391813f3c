"""Builds the HIP libraries for gfx950 with hipcc, in-tree, and finds them again.

One "core" library per element type (matrix products, norms, rotation and cache write,
embedding, sampling) and one attention library per element type and head-size tile.  A
library is rebuilt when the hash of its sources and flags differs from the stamp beside it,
so a fresh checkout compiles at its first call exactly the libraries the model at hand
needs, and prints a line now and then while it does.
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
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc")
CSRC = os.path.normpath(CSRC)
ARCH = "gfx950"
FLAGS = ["-O3", f"--offload-arch={ARCH}", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-inline-asm"]
ELEM_DEFINE = {"bf16": "MS_ELEM_BF16", "f16": "MS_ELEM_F16", "f32": "MS_ELEM_F32"}
CORE_SOURCES = ["errors.hip", "gemm.hip", "skinny.hip", "elementwise.hip", "sampling.hip"]
ATTENTION_TILES = (1, 2, 3, 4, 6, 8, 12, 16)  # head-size tiles in units of 16

_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def attention_tile_for(head_dim: int) -> int:
    if head_dim % 16 or head_dim <= 0:
        raise BuildError(f"head size {head_dim} is not a positive multiple of 16")
    for nd in ATTENTION_TILES:
        if nd * 16 >= head_dim:
            return nd
    raise BuildError(f"head size {head_dim} exceeds the largest attention tile of {ATTENTION_TILES[-1] * 16}")


def _lib_dir() -> str:
    """In-tree ``machserve_amd/_lib``; a per-user temporary folder if the tree is read-only."""
    d = os.path.normpath(os.path.join(CSRC, "..", "_lib"))
    try:
        os.makedirs(d, exist_ok=True)
        if os.access(d, os.W_OK):
            return d
    except OSError:
        pass
    d = os.path.join(tempfile.gettempdir(), f"machserve_amd_lib_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


def _sources_of(kind: str):
    if kind == "core":
        return list(CORE_SOURCES)
    return ["errors.hip", "attention.hip"]


def _spec(kind: str, elem: str, nd: int | None):
    defines = [ELEM_DEFINE[elem]]
    name = f"ms_{kind}_{elem}"
    if kind == "attention":
        defines.append(f"MS_ATTN_ND={nd}")
        name += f"_nd{nd}"
    return name, _sources_of(kind), defines


def _digest(sources, defines) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + defines).encode())
    headers = {f for f in os.listdir(CSRC) if f.endswith((".cuh", ".h"))}
    for f in sorted(set(sources) | headers):
        with open(os.path.join(CSRC, f), "rb") as fh:   # a source outside the folder is given by its full path
            h.update(os.path.basename(f).encode())
            h.update(fh.read())
    return h.hexdigest()


def _say(msg: str) -> None:
    print(f"[machserve_amd build] {msg}", file=sys.stderr, flush=True)


def _run_with_heartbeat(cmd, what: str) -> None:
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def beat():
        while not done.wait(20.0):
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")

    th = threading.Thread(target=beat, daemon=True)
    th.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise BuildError(f"{what}: the compiler failed\n$ {' '.join(cmd)}\n{out}")


_locks: dict = {}


def _lock_of(name: str) -> threading.Lock:
    with _lock:
        return _locks.setdefault(name, threading.Lock())


def ensure_library(kind: str, elem: str, nd: int | None = None, force: bool = False) -> str:
    """Path of the built library; compiles it first if it is missing or stale (or ``force``)."""
    name, sources, defines = _spec(kind, elem, nd)
    return _ensure(name, sources, defines, force)


def ensure_extra_library(name: str, elem: str, source: str, force: bool = False) -> str:
    """A library of the caller's own: one HIP source given by its path, which may include this package's
    headers and is linked with its error channel; built with the same flags and kept beside the others."""
    return _ensure(f"{name}_{elem}", ["errors.hip", os.path.abspath(source)], [ELEM_DEFINE[elem]], force)


def _ensure(name: str, sources, defines, force: bool) -> str:
    libdir = _lib_dir()
    so = os.path.join(libdir, f"lib{name}.so")
    stamp = so + ".stamp"
    digest = _digest(sources, defines)
    with _lock_of(name):
        if not force and os.path.exists(so) and os.path.exists(stamp):
            with open(stamp) as f:
                if f.read().strip() == digest:
                    return so
        hipcc = _hipcc()
        objdir = os.path.join(libdir, "obj", name)
        os.makedirs(objdir, exist_ok=True)
        _say(f"compiling {name} for {ARCH} ({len(sources)} files)")
        t0 = time.time()
        objs = [os.path.join(objdir, os.path.basename(s).replace(".hip", ".o")) for s in sources]

        def one(pair):
            src, obj = pair
            cmd = [hipcc, *FLAGS, *[f"-D{d}" for d in defines], f"-I{CSRC}", "-c", os.path.join(CSRC, src), "-o", obj]
            _run_with_heartbeat(cmd, f"{name}/{os.path.basename(src)}")

        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            list(pool.map(one, zip(sources, objs)))
        tmp = so + f".tmp{os.getpid()}"
        _run_with_heartbeat([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs], f"link {name}")
        os.replace(tmp, so)
        with open(stamp, "w") as f:
            f.write(digest)
        _say(f"built {os.path.basename(so)} in {time.time() - t0:.0f} s")
        return so


HOST_SOURCES = [os.path.join("host", f) for f in ("module.cpp", "cache.hpp", "scheduler.hpp")]  # the first is compiled
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall"]
_host_module = None


def ensure_host_module(force: bool = False):
    """The host runtime (pools, cache manager, step buffer builder) as an imported module; it is
    compiled from ``csrc/host/module.cpp`` with the C++ compiler and pybind11 when missing or stale."""
    global _host_module
    import importlib.util
    import sysconfig
    with _lock_of("ms_host"):
        if _host_module is not None and not force:
            return _host_module
        src = os.path.join(CSRC, HOST_SOURCES[0])
        libdir = _lib_dir()
        so = os.path.join(libdir, "ms_host" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
        stamp = so + ".stamp"
        h = hashlib.sha256(" ".join(HOST_FLAGS).encode())
        for f in HOST_SOURCES:
            with open(os.path.join(CSRC, f), "rb") as fh:
                h.update(fh.read())
        digest = h.hexdigest()
        fresh = False
        if not force and os.path.exists(so) and os.path.exists(stamp):
            with open(stamp) as f:
                fresh = f.read().strip() == digest
        if not fresh:
            try:
                import pybind11
            except ImportError as e:
                raise BuildError("pybind11 is needed to build the host runtime") from e
            cxx = next((c for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"))
                        if c), None)
            if cxx is None:
                raise BuildError("no C++ compiler found (looked at $CXX, g++, c++, clang++): the host runtime cannot be built")
            _say("compiling the host runtime (ms_host)")
            t0 = time.time()
            tmp = so + f".tmp{os.getpid()}"
            cmd = [cxx, *HOST_FLAGS, f"-I{pybind11.get_include()}", f"-I{sysconfig.get_paths()['include']}", src, "-o", tmp]
            _run_with_heartbeat(cmd, "ms_host")
            os.replace(tmp, so)
            with open(stamp, "w") as f:
                f.write(digest)
            _say(f"built {os.path.basename(so)} in {time.time() - t0:.0f} s")
        spec = importlib.util.spec_from_file_location("ms_host", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _host_module = mod
        return mod


def build_all(force: bool = True, workers: int = 4) -> list:
    """Every library of both element types and the host runtime (what ``__graft_entry__.build`` calls)."""
    ensure_host_module(force=force)
    jobs = []
    for elem in ELEM_DEFINE:
        jobs.append(("core", elem, None))
        for nd in ATTENTION_TILES:
            jobs.append(("attention", elem, nd))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        return list(pool.map(lambda j: ensure_library(*j, force=force), jobs))
