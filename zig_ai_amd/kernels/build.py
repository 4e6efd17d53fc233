"""Compiling the sources under ``csrc/`` and loading the result: the HIP kernels
for gfx950 with hipcc, the host-side bookkeeping (``host.cpp``) with the C++
compiler.

Every ``<name>.hip`` / ``<name>.cpp`` becomes ``lib<name>.so`` in ``zig_ai_amd/_lib`` (or, when
the package folder cannot be written, in a per-user folder under the system's
temporary directory).  A library is compiled the first time something needs it
and it is not there, or when its sources have changed since it was built;
``build_all(force=True)`` compiles everything regardless.  While compiling, a
line is printed now and then so that a first call does not look hung.
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
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Iterable, List, Optional

PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(PACKAGE_DIR, "csrc")
ARCH = "gfx950"
SOURCES = ("norm", "gemm", "gemm_rows64", "rope_kv", "attention", "shortconv", "activation",
           "sampling", "blaslt", "calibrate")
HOST_SOURCES = ("host", "plain")    # plain C++, no device code: usable without a GPU or ROCm
ALL_SOURCES = SOURCES + HOST_SOURCES
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden"]
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

EXTRA_FLAGS = {"blaslt": ["-lhipblaslt"]}   # host code around the GEMM library, no kernels
# headers a source includes beside common.h
EXTRA_HEADERS = {"sampling": ["no_alloc.h"], "rope_kv": ["rope_math.h"], "attention": ["rope_math.h"]}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[zig_ai_amd] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def find_cxx() -> Optional[str]:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"),
                 shutil.which("clang++"), find_hipcc()):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _source_of(name: str) -> str:
    return os.path.join(CSRC_DIR, name + (".cpp" if name in HOST_SOURCES else ".hip"))


def _lib_dirs() -> List[str]:
    """Folders that may hold built libraries, in order of preference."""
    dirs = [os.path.join(PACKAGE_DIR, "_lib")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"zig_ai_amd-{uid}", "_lib"))
    return dirs


def _writable_lib_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}-{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError("no writable folder for compiled kernels: tried " + ", ".join(_lib_dirs()))


def source_digest(name: str) -> str:
    h = hashlib.sha256()
    host = name in HOST_SOURCES
    headers = ([] if host else ["common.h"]) + EXTRA_HEADERS.get(name, [])
    for path in [os.path.join(CSRC_DIR, h) for h in headers] + [_source_of(name)]:
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join((CXX_FLAGS if host else HIPCC_FLAGS) + EXTRA_FLAGS.get(name, [])).encode())
    return h.hexdigest()


def _find_built(name: str) -> Optional[str]:
    """Path of an up-to-date library, or None."""
    want = source_digest(name)
    for d in _lib_dirs():
        so = os.path.join(d, f"lib{name}.so")
        tag = so + ".digest"
        if os.path.isfile(so) and os.path.isfile(tag):
            try:
                with open(tag, "r") as f:
                    if f.read().strip() == want:
                        return so
            except OSError:
                pass
    return None


def _find_stale(name: str) -> Optional[str]:
    for d in _lib_dirs():
        so = os.path.join(d, f"lib{name}.so")
        if os.path.isfile(so):
            return so
    return None


def compile_one(name: str) -> str:
    host = name in HOST_SOURCES
    src = _source_of(name)
    if not os.path.isfile(src):
        raise KernelBuildError(f"{src} does not exist")
    if host:
        cxx = find_cxx()
        if cxx is None:
            raise KernelBuildError(
                f"lib{name}.so is not built and no C++ compiler was found "
                "(looked at $CXX, g++, c++, clang++ and hipcc)")
        flags = CXX_FLAGS + (["-x", "c++"] if os.path.basename(cxx).startswith("hipcc") else [])
    else:
        cxx = find_hipcc()
        if cxx is None:
            raise KernelBuildError(
                f"kernel library lib{name}.so is not built and hipcc was not found "
                "(looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")
        flags = HIPCC_FLAGS
    out_dir = _writable_lib_dir()
    so = os.path.join(out_dir, f"lib{name}.so")
    tmp = os.path.join(out_dir, f".lib{name}.{os.getpid()}.{threading.get_ident()}.so")
    cmd = [cxx] + flags + ["-I", CSRC_DIR, "-o", tmp, src] + EXTRA_FLAGS.get(name, [])
    what = os.path.basename(src)
    env = dict(os.environ)
    home = env.get("HOME", "")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        env["HOME"] = tempfile.gettempdir()   # the compiler wants a writable HOME
    start = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    output: List[str] = []

    def drain() -> None:
        assert proc.stdout is not None
        for line in proc.stdout:
            output.append(line)

    reader = threading.Thread(target=drain, daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=15)
            break
        except subprocess.TimeoutExpired:
            _say(f"still compiling {what} ({time.time() - start:.0f} s)")
    reader.join()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        text = "".join(l for l in output if "packed-fp32-ops" not in l)
        raise KernelBuildError(f"{os.path.basename(cxx)} failed on {what} (exit {proc.returncode}):\n{text}")
    os.replace(tmp, so)
    with open(so + ".digest.tmp", "w") as f:
        f.write(source_digest(name))
    os.replace(so + ".digest.tmp", so + ".digest")
    _say(f"compiled {what} in {time.time() - start:.1f} s -> {so}")
    return so


def build_all(names: Iterable[str] = ALL_SOURCES, force: bool = False, jobs: int = 4) -> Dict[str, str]:
    """Compile the named sources (all by default); with ``force`` also those
    that are up to date.  Returns ``{name: path}``."""
    names = list(names)
    todo = [n for n in names if force or _find_built(n) is None]
    paths = {n: _find_built(n) for n in names if n not in todo}
    if todo:
        _say(f"compiling {len(todo)} source(s) (kernels for {ARCH}): {', '.join(todo)}")
        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as pool:
            for n, p in zip(todo, pool.map(compile_one, todo)):
                paths[n] = p
    return paths


def load(name: str) -> ctypes.CDLL:
    """The library of ``csrc/<name>.hip`` (or ``.cpp``), compiled first if need be."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        path = _find_built(name)
        if path is None:
            stale = _find_stale(name)
            if stale is not None and (find_cxx() if name in HOST_SOURCES else find_hipcc()) is None:
                raise KernelBuildError(
                    f"{stale} was built from other sources than the ones present and no "
                    "compiler is available to rebuild it")
            path = compile_one(name)
        lib = ctypes.CDLL(path)
        _loaded[name] = lib
        return lib
