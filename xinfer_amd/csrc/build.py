"""Builds the two native libraries in-tree and loads them.

`libxinfer_hip.so`  : the gfx950 kernels (hipcc), one object per .hip file.
`libxinfer_host.so` : cache manager, batch builder and scheduler (g++).

A library is rebuilt when it is missing or older than the digest of its sources; a
first call in a fresh checkout therefore compiles what is needed and prints a line per
file meanwhile.  If the package folder cannot be written, a per-user folder under the
system's temporary directory is used instead.  Nothing falls back to another
implementation: a library that cannot be built or loaded is an error.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.dirname(_HERE)
KERNEL_DIR = os.path.join(_HERE, "kernels")
HOST_DIR = os.path.join(_HERE, "host")

HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # no packed-FP32 instructions in the generated code: some of their forms have given wrong results on gfx950
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra"]


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[xinfer_amd build] {msg}", file=sys.stderr, flush=True)


def _sources(folder: str, exts) -> List[str]:
    return sorted(os.path.join(folder, f) for f in os.listdir(folder) if f.endswith(tuple(exts)))


def _digest(paths: List[str], flags: List[str]) -> str:
    h = hashlib.sha256()
    h.update(" ".join(flags).encode())
    for p in paths:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _lib_dir() -> str:
    """In-tree `_lib/` if it can be written, else a per-user temporary folder."""
    d = os.path.join(_PKG, "_lib")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        # a folder of this user alone: nobody else may plant a library there
        base = os.path.join(tempfile.gettempdir(), f"xinfer_amd-{os.getuid()}")
        try:
            os.makedirs(base, mode=0o700, exist_ok=True)
            st = os.stat(base)
            if st.st_uid != os.getuid() or (st.st_mode & 0o022):
                raise OSError("not ours")
        except OSError:
            base = tempfile.mkdtemp(prefix="xinfer_amd-")
        d = os.path.join(base, "_lib")
        os.makedirs(d, exist_ok=True)
        return d


def _find(tool: str, extra: List[str]) -> Optional[str]:
    p = shutil.which(tool)
    if p:
        return p
    for c in extra:
        if os.path.isfile(c) and os.access(c, os.X_OK):
            return c
    return None


def _run(cmd: List[str], what: str) -> None:
    env = dict(os.environ)
    home = env.get("HOME")
    if not home or not os.path.isdir(home) or not os.access(home, os.W_OK):
        env["HOME"] = tempfile.gettempdir()            # hipcc wants a HOME it can write its caches to
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if r.returncode != 0:
        raise BuildError(f"{what} failed (exit {r.returncode}):\n{' '.join(cmd)}\n{r.stdout}")


def _current(lib: str, digest: str) -> bool:
    tag = lib + ".digest"
    if not (os.path.isfile(lib) and os.path.isfile(tag)):
        return False
    with open(tag, "r") as f:
        return f.read().strip() == digest


def _stamp(lib: str, digest: str) -> None:
    with open(lib + ".digest", "w") as f:
        f.write(digest)


def build_kernels(force: bool = False) -> str:
    srcs = _sources(KERNEL_DIR, (".hip",))
    deps = srcs + _sources(KERNEL_DIR, (".h",))
    digest = _digest(deps, HIP_FLAGS)
    # a library shipped in-tree wins over the temporary folder
    for d in (os.path.join(_PKG, "_lib"), None):
        cand = os.path.join(d if d else _lib_dir(), "libxinfer_hip.so")
        if not force and _current(cand, digest):
            return cand
    out_dir = _lib_dir()
    lib = os.path.join(out_dir, "libxinfer_hip.so")
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"])
    if hipcc is None:
        raise BuildError("hipcc not found: the gfx950 kernel library cannot be built")
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    _say(f"compiling {len(srcs)} HIP sources for gfx950 into {lib}")
    t0 = time.time()

    headers = _sources(KERNEL_DIR, (".h",))

    def one(src: str) -> str:
        # an object is kept while its source, the headers and the flags are what it was made from
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        own = _digest([src] + headers, HIP_FLAGS)
        if not force and _current(obj, own):
            return obj
        t = time.time()
        _run([hipcc, *HIP_FLAGS, "-I", KERNEL_DIR, "-c", src, "-o", obj], f"hipcc {os.path.basename(src)}")
        _stamp(obj, own)
        _say(f"  {os.path.basename(src)} done in {time.time() - t:.0f}s")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(workers) as ex:
        objs = list(ex.map(one, srcs))
    tmp = lib + f".tmp{os.getpid()}"
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", tmp], "link libxinfer_hip.so")
    os.replace(tmp, lib)
    _stamp(lib, digest)
    _say(f"kernel library ready after {time.time() - t0:.0f}s")
    return lib


def build_host(force: bool = False) -> str:
    srcs = _sources(HOST_DIR, (".cpp",))
    deps = srcs + _sources(HOST_DIR, (".h",))
    digest = _digest(deps, HOST_FLAGS)
    for d in (os.path.join(_PKG, "_lib"), None):
        cand = os.path.join(d if d else _lib_dir(), "libxinfer_host.so")
        if not force and _current(cand, digest):
            return cand
    out_dir = _lib_dir()
    lib = os.path.join(out_dir, "libxinfer_host.so")
    cxx = _find("g++", ["/usr/bin/g++", "/usr/bin/c++", "/opt/rocm/llvm/bin/clang++"])
    if cxx is None:
        raise BuildError("no C++ compiler found: the host runtime library cannot be built")
    _say(f"compiling the host runtime into {lib}")
    tmp = lib + f".tmp{os.getpid()}"
    _run([cxx, *HOST_FLAGS, "-shared", "-I", HOST_DIR, *srcs, "-o", tmp], "g++ host runtime")
    os.replace(tmp, lib)
    _stamp(lib, digest)
    return lib


_loaded: Dict[str, ctypes.CDLL] = {}


def load_kernels() -> ctypes.CDLL:
    if "hip" not in _loaded:
        path = build_kernels()
        try:
            _loaded["hip"] = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"the gfx950 kernel library {path} cannot be loaded: {e}") from e
    return _loaded["hip"]


def load_host() -> ctypes.CDLL:
    if "host" not in _loaded:
        path = build_host()
        try:
            _loaded["host"] = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"the host runtime library {path} cannot be loaded: {e}") from e
    return _loaded["host"]


def build_all(force: bool = True) -> None:
    build_host(force=force)
    build_kernels(force=force)


if __name__ == "__main__":
    build_all(force=True)
