"""Compiles the HIP sources under ``csrc/`` into one shared library for gfx950.

``hipcc`` is called directly, one process per source file, then once to link.
The library is written next to the sources (``csrc/_build/``) when that folder
can be written, else into a per-user folder under the system's temporary
directory, so that a read-only checkout still works.
"""

from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libfmsamd.so"
DIGEST_NAME = "digest.txt"
ARCH = "gfx950"

# -packed-fp32-ops: keep the compiler from forming packed float32 instructions.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-pass-failed",
]


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_digest() -> str:
    h = hashlib.sha256()
    for path in sources() + sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    """Where a built library may be, in the order of preference."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [os.path.join(CSRC, "_build"), os.path.join(tempfile.gettempdir(), f"fmsamd_build_{uid}")]


def find_library() -> Optional[str]:
    for folder in build_dirs():
        path = os.path.join(folder, LIB_NAME)
        if os.path.isfile(path):
            return path
    return None


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc was not found: the kernels of this library are HIP sources and must be compiled")


def _say(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[fms_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path.  Always compiles."""
    hipcc = hipcc_path()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable build folder among {build_dirs()}")
    srcs = sources()
    start = time.time()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}", verbose)

    # objects go to a folder of this process, so that two processes building at once do not write one file
    obj_dir = tempfile.mkdtemp(prefix=f".obj{os.getpid()}_", dir=out_dir)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}")
        _say(f"compiled {os.path.basename(src)} ({time.time() - start:.0f} s)", verbose)
        return obj

    try:
        digest = source_digest()
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
            objs = list(pool.map(compile_one, srcs))
        tmp = os.path.join(obj_dir, LIB_NAME)
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed to link:\n{proc.stdout}")
        lib = os.path.join(out_dir, LIB_NAME)
        os.replace(tmp, lib)
        digest_tmp = os.path.join(obj_dir, DIGEST_NAME)
        with open(digest_tmp, "w") as f:
            f.write(digest)
        os.replace(digest_tmp, os.path.join(out_dir, DIGEST_NAME))
    finally:
        shutil.rmtree(obj_dir, ignore_errors=True)
    _say(f"linked {lib} ({time.time() - start:.0f} s)", verbose)
    return lib


def library_is_current(lib: str) -> bool:
    """True if the library's folder records the digest of the sources as they are now."""
    try:
        with open(os.path.join(os.path.dirname(lib), DIGEST_NAME)) as f:
            return f.read().strip() == source_digest()
    except OSError:
        return False


def ensure_built(verbose: bool = True) -> str:
    """The path of a library built from the sources as they are now.  A built copy whose recorded digest
    matches is used as it is; otherwise the library is compiled.  A copy that is older than the sources is
    never used: if it cannot be replaced (no compiler, no writable folder) this raises."""
    for folder in build_dirs():
        lib = os.path.join(folder, LIB_NAME)
        if os.path.isfile(lib) and library_is_current(lib):
            return lib
    stale = find_library()
    if stale is not None:
        _say(f"{stale} was built from other sources than the present ones: compiling again", verbose)
    try:
        return build(verbose)
    except Exception as err:
        if stale is not None:
            raise RuntimeError(f"{stale} does not match the present sources and could not be rebuilt: {err}") from err
        raise


if __name__ == "__main__":
    print(build())
