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
ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


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


def library_path() -> str:
    """The built library: in-tree if it is there, else the fallback location."""
    in_tree = os.path.join(HERE, LIB_NAME)
    if os.path.isfile(in_tree):
        return in_tree
    return os.path.join(_fallback_dir(), LIB_NAME)


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

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc] + FLAGS + ["-c", os.path.join(HERE, src), "-o", obj]
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
    build()
