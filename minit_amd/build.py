"""Builds the HIP shared library for gfx950 with hipcc.

The reference compiles CUDA source strings at run time with ``nvcc -shared`` into
``~/.minit/cached/<md5>/library.so`` (minit/cuda/compiler.py:9-25,
minit/compiler/cache.py:8-28).  Here the sources are files under ``csrc/`` and
the library is built ahead of time, in-tree, next to this module:
``python -m minit_amd.build``.  Object files are cached by a content hash of the
source, the headers and the flags so an unchanged file is not recompiled.
"""
import hashlib
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libminit_hip.so")

ARCH = "gfx950"
# -packed-fp32-ops is switched off on purpose: hipcc otherwise forms packed fp32
# instructions from scalar float code.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _digest(src: str) -> str:
    h = hashlib.md5()
    h.update(" ".join(HIPCC_FLAGS).encode())
    with open(os.path.join(CSRC, src), "rb") as f:
        h.update(f.read())
    for root in (CSRC, INCLUDE):
        for name in sorted(os.listdir(root)):
            if name.endswith(".h"):
                with open(os.path.join(root, name), "rb") as f:
                    h.update(f.read())
    return h.hexdigest()[:12]


def _compile_one(hipcc: str, src: str, force: bool, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, f"{os.path.splitext(src)[0]}.{_digest(src)}.o")
    if os.path.exists(obj) and not force:
        return obj
    tmp = obj + ".tmp"
    cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, obj)  # a cached object is either absent or complete
    return obj


def build(force: bool = False, verbose: bool = True, jobs: int = 4) -> str:
    """Compiles every ``csrc/*.hip`` for gfx950 and links ``libminit_hip.so``.

    One builder at a time (a file lock on the object directory, as the reference
    guards its kernel cache, minit/compiler/cache.py:8-28)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    from filelock import FileLock
    with FileLock(os.path.join(OBJ_DIR, ".lock")):
        return _build_locked(force, verbose, jobs)


def _build_locked(force: bool, verbose: bool, jobs: int) -> str:
    hipcc = find_hipcc()
    srcs = sources()
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(lambda s: _compile_one(hipcc, s, force, verbose), srcs))
    keep = set(objs)
    for name in os.listdir(OBJ_DIR):
        path = os.path.join(OBJ_DIR, name)
        if name.endswith(".o") and path not in keep:
            os.remove(path)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
