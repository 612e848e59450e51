"""Builds the gfx950 kernel library from the .hip sources beside this file.

`build()` always compiles; `library_path()` says where the result lives. The
library is built in-tree (csrc/libimparo_hip.so); when the tree is not
writable it goes to a per-user folder under the system temp directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libimparo_hip.so"
HOST_LIB_NAME = "libimparo_host.so"     # the host runtime (no GPU code): csrc/host/*.cpp
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _hash_of(paths: List[str]) -> str:
    h = hashlib.sha256()
    for path in sorted(paths):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def source_hash() -> str:
    """A hash of everything the kernel library is compiled from. The library
    carries the hash of the sources it was built from (imparo_hip_source_hash),
    so that a library older than its sources is noticed when it is loaded."""
    return _hash_of([os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith((".hip", ".h"))])


def host_source_hash() -> str:
    src_dir = os.path.join(HERE, "host")
    return _hash_of([os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith((".cpp", ".h"))])


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc was not found (looked on PATH and in /opt/rocm/bin); "
                       "the gfx950 kernel library cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _fallback_dir() -> str:
    tag = hashlib.sha256(HERE.encode()).hexdigest()[:12]
    return os.path.join(tempfile.gettempdir(), f"imparo_amd_build_{os.getuid()}_{tag}")


def library_path(name: str = LIB_NAME) -> str:
    """The built library: in-tree if it is there, else the fallback location."""
    in_tree = os.path.join(HERE, name)
    if os.path.isfile(in_tree):
        return in_tree
    return os.path.join(_fallback_dir(), name)


def host_library_path() -> str:
    return library_path(HOST_LIB_NAME)


def build_host(verbose: bool = True) -> str:
    """Compiles the host runtime library with the C++ compiler."""
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if cxx is None:
        for cand in ("/opt/rocm/lib/llvm/bin/clang++", "/opt/rocm/llvm/bin/clang++"):
            if os.path.isfile(cand):
                cxx = cand
    if cxx is None:
        raise RuntimeError("no C++ compiler was found (g++, c++, clang++); the host runtime cannot be built")
    out_dir = HERE if _writable(os.path.join(HERE, "_build")) else _fallback_dir()
    os.makedirs(out_dir, exist_ok=True)
    src_dir = os.path.join(HERE, "host")
    srcs = sorted(os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith(".cpp"))
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    stamp = f'-DIMPARO_SOURCE_HASH="{host_source_hash()}"'
    proc = subprocess.run([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", stamp, "-I", src_dir] + srcs + ["-o", tmp],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {HOST_LIB_NAME} failed:\n{proc.stderr}")
    os.replace(tmp, lib)
    if verbose:
        _say(f"built {lib}")
    return lib


def _say(msg: str) -> None:
    print(f"[imparo_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compiles every .hip source for gfx950 and links the shared library."""
    hipcc = _hipcc()
    out_dir = HERE if _writable(os.path.join(HERE, "_build")) else _fallback_dir()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    if verbose:
        _say(f"compiling {len(srcs)} sources for {ARCH} into {out_dir}")

    stamp = f'-DIMPARO_SOURCE_HASH="{source_hash()}"'

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc] + FLAGS + [stamp, "-c", os.path.join(HERE, src), "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stderr}")
        if verbose:
            _say(f"compiled {src}")
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    proc = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC"] + objs + ["-o", tmp],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{proc.stderr}")
    os.replace(tmp, lib)
    if verbose:
        _say(f"linked {lib}")
    return lib


if __name__ == "__main__":
    build_host()
    build()
