"""Builds the HIP sources of this folder into one shared library for gfx950
and the C++ host runtime (host/) into another, and loads them. The library's file name carries a hash of the sources and flags,
so a stale build is never loaded: when no file of the current hash exists, it
is compiled at the first call (a line is printed for every file meanwhile)."""
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
from pathlib import Path

from ..errors import AlofaError

HERE = Path(__file__).resolve().parent
ARCH = "gfx950"
# -packed-fp32-ops off: the compiler must not form packed float instructions
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

_lib = None


def sources() -> list:
    return sorted(HERE.glob("*.hip"))


def _hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for p in sorted(list(HERE.glob("*.hip")) + list(HERE.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()[:12]


def _lib_name() -> str:
    return f"libalofa_hip_{_hash()}.so"


HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-fopenmp"]      # (threads share out independent outputs of the plain path only)
_host = None


def host_sources() -> list:
    return sorted((HERE / "host").glob("*.cpp"))


def _host_name() -> str:
    h = hashlib.sha256(" ".join(HOST_FLAGS).encode())
    for p in host_sources():
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return f"libalofa_host_{h.hexdigest()[:12]}.so"


def find_built_host():
    for d in _candidate_dirs():
        if (d / _host_name()).is_file():
            return d / _host_name()
    return None


def build_host(force: bool = False) -> Path:
    """Compile the host runtime (plain C++, no GPU code) with the system compiler."""
    if not force:
        found = find_built_host()
        if found:
            return found
    cxx = next((c for c in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")) if c), None)
    if cxx is None:
        raise AlofaError("not_initialized", "no C++ compiler was found; the host runtime cannot be built")
    target_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if target_dir is None:
        raise AlofaError("io", "no writable folder for the built library", f"tried={[str(d) for d in _candidate_dirs()]}")
    out = target_dir / _host_name()
    tmp = target_dir / (out.name + f".tmp{os.getpid()}")
    _say(f"compiling the host runtime into {target_dir}")
    r = subprocess.run([cxx, *HOST_FLAGS, "-o", str(tmp), *map(str, host_sources())], capture_output=True, text=True)
    if r.returncode != 0:
        raise AlofaError("io", "compiling the host runtime failed", r.stderr[-4000:])
    os.replace(tmp, out)
    for old in target_dir.glob("libalofa_host_*.so"):
        if old != out:
            try:
                old.unlink()
            except OSError:
                pass
    return out


def load_host() -> ctypes.CDLL:
    """The host runtime (pool, cache accounting, scheduler); built first when missing."""
    global _host
    if _host is None:
        path = find_built_host() or build_host()
        try:
            _host = ctypes.CDLL(str(path))
        except OSError as e:
            raise AlofaError("not_initialized", "the host runtime cannot be loaded", f"path={path} reason={e}") from None
        c = ctypes
        _host.alofa_host_last_error.restype = c.c_char_p
        for name in ("alofa_pool_new", "alofa_cache_new", "alofa_cache_pool", "alofa_sched_new"):
            getattr(_host, name).restype = c.c_void_p
        for name in ("alofa_cache_length", "alofa_sched_scalar", "alofa_sched_scalar_of"):
            getattr(_host, name).restype = c.c_int64
    return _host


def _candidate_dirs() -> list:
    out = [HERE]
    base = Path(os.environ.get("TMPDIR") or tempfile.gettempdir())
    out.append(base / f"alofa_amd_build_{os.getuid()}")
    return out


def find_built():
    name = _lib_name()
    for d in _candidate_dirs():
        if (d / name).is_file():
            return d / name
    return None


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and Path(c).exists():
            return c
    raise AlofaError("not_initialized", "hipcc was not found; the HIP library cannot be built", "looked in PATH and /opt/rocm/bin")


def _say(text: str) -> None:
    print(f"[alofa_amd build] {text}", file=sys.stderr, flush=True)


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe_{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def build(force: bool = False) -> Path:
    """Compile every .hip file and link them. Returns the library's path."""
    if not force:
        found = find_built()
        if found:
            return found
    hipcc = _hipcc()
    target_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if target_dir is None:
        raise AlofaError("io", "no writable folder for the built library", f"tried={[str(d) for d in _candidate_dirs()]}")
    obj_dir = target_dir / "_build"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    _say(f"compiling {len(srcs)} HIP files for {ARCH} into {target_dir}")
    t0 = time.time()

    def compile_one(src: Path):
        obj = obj_dir / (src.stem + ".o")
        r = subprocess.run([hipcc, *FLAGS, "-c", str(src), "-o", str(obj)], capture_output=True, text=True)
        if r.returncode != 0:
            raise AlofaError("io", "hipcc failed", f"file={src.name}\n{r.stderr[-4000:]}")
        _say(f"  {src.name} done ({time.time() - t0:.0f}s)")
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    out = target_dir / _lib_name()
    tmp = target_dir / (out.name + f".tmp{os.getpid()}")
    r = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise AlofaError("io", "linking the HIP library failed", r.stderr[-4000:])
    os.replace(tmp, out)
    for old in target_dir.glob("libalofa_hip_*.so"):
        if old != out:
            try:
                old.unlink()
            except OSError:
                pass
    _say(f"built {out.name} in {time.time() - t0:.0f}s")
    return out


def load() -> ctypes.CDLL:
    """The loaded library; built first when no current build exists. There is
    no fallback: without the library nothing runs."""
    global _lib
    if _lib is None:
        # torch first: its HIP runtime must be the one in the process, so that the
        # library shares it (and torch's streams and memory) instead of loading a second copy
        import torch  # noqa: F401
        path = find_built() or build()
        try:
            _lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise AlofaError("not_initialized", "the HIP library cannot be loaded", f"path={path} reason={e}") from None
        _lib.alofa_last_error.restype = ctypes.c_char_p
    return _lib
