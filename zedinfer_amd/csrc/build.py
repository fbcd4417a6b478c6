"""Building and finding the HIP kernel library.

The kernels are plain HIP with an ``extern "C"`` interface, compiled for gfx950
with hipcc into one shared library that Python loads with ctypes: no torch
headers, so a cold build takes well under a minute on a few cores.  The library
is keyed by a hash of its sources and flags.  It is looked for, and built, in
``zedinfer_amd/_lib`` when that folder can be written, else in a per-user
folder under the temporary directory.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import List, Optional

CSRC = os.path.dirname(os.path.abspath(__file__))
PACKAGE = os.path.dirname(CSRC)
LIB_NAME = "libzedinfer_hip.so"
ARCH = "gfx950"

# -packed-fp32-ops is switched off: hipcc would otherwise fuse float pairs into
# packed instructions on its own.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
]
# More flags for hipcc from the environment (a probe build, e.g. -DDL_TIMING); they go into the library's hash.
FLAGS += os.environ.get("ZEDINFER_AMD_EXTRA_FLAGS", "").split()
# The library matrix product (gemm_lt.hip) is hipBLASLt's.
LINK_LIBS = ["-lhipblaslt"]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def headers() -> List[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + LINK_LIBS).encode())
    for f in sources() + headers():
        h.update(f.encode())
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


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


def lib_dirs() -> List[str]:
    """Folders searched for the library, in order."""
    dirs = [os.path.join(PACKAGE, "_lib")]
    env = os.environ.get("ZEDINFER_AMD_LIB_DIR")
    if env:
        dirs.insert(0, env)
    dirs.append(os.path.join(tempfile.gettempdir(), f"zedinfer_amd-{os.getuid()}"))
    return dirs


def _hash_of(lib: str) -> Optional[str]:
    try:
        with open(lib + ".hash") as f:
            return f.read().strip()
    except OSError:
        return None


def find_library(require_current: bool = True) -> Optional[str]:
    want = source_hash()
    stale = None
    for d in lib_dirs():
        lib = os.path.join(d, LIB_NAME)
        if os.path.isfile(lib):
            if _hash_of(lib) == want:
                return lib
            stale = stale or lib
    return None if require_current else stale


def hipcc_path() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _say(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[zedinfer_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True, force: bool = True, jobs: Optional[int] = None) -> str:
    """Compile every kernel source and link the library; returns its path."""
    if not force:
        lib = find_library()
        if lib:
            return lib
    hipcc = hipcc_path()
    if hipcc is None:
        raise RuntimeError("hipcc not found: the HIP kernel library cannot be built "
                           "(set HIPCC or install ROCm under /opt/rocm)")
    out_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library among: " + ", ".join(lib_dirs()))
    want = source_hash()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    _say(f"compiling {len(srcs)} kernel sources for {ARCH} with {jobs} jobs into {out_dir}", verbose)
    t0 = time.time()
    done = threading.Event()

    def heartbeat():
        while not done.wait(15.0):
            _say(f"still compiling ({time.time() - t0:.0f} s)", verbose)

    hb = threading.Thread(target=heartbeat, daemon=True)
    hb.start()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc] + FLAGS + ["-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
        _say(f"compiled {src} ({time.time() - t0:.0f} s)", verbose)
        return obj

    try:
        with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
            objs = list(ex.map(compile_one, srcs))
        tmp_lib = os.path.join(obj_dir, LIB_NAME + f".{os.getpid()}")
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp_lib] + objs + LINK_LIBS
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"linking the kernel library failed:\n{r.stderr[-4000:]}")
    finally:
        done.set()
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(tmp_lib, lib)
    with open(lib + ".hash", "w") as f:
        f.write(want)
    _say(f"built {lib} in {time.time() - t0:.0f} s", verbose)
    return lib


def ensure_library(verbose: bool = True) -> str:
    """The path of a library that matches the sources, building it when there is none."""
    lib = find_library()
    if lib:
        return lib
    if hipcc_path() is None:
        stale = find_library(require_current=False)
        raise RuntimeError(
            "the HIP kernel library is missing" + (f" (a stale one is at {stale})" if stale else "") +
            " and hipcc is not available to build it; run __graft_entry__.build() where ROCm is installed")
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
