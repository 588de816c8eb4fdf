"""Compile the HIP sources for gfx950 into one shared library with plain ``hipcc``.

No torch headers are involved: the kernels take raw device pointers and a stream, and the
Python side binds them with ``ctypes``.  The library lands beside the sources
(``sharpinference_amd/csrc/_build/libsharpi_hip.so``); if that folder cannot be written the
build goes to a per-user folder under the system's temporary directory.  A stamp of the
sources' hash sits next to the library, so a stale build is noticed and redone.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

CSRC_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libsharpi_hip.so"
ARCH = "gfx950"

HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    f"--offload-arch={ARCH}",
    "-fvisibility=hidden",
    "-Wno-unused-result",
    # packed FP32 instructions (v_pk_*_f32) are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> List[str]:
    return sorted(f for f in os.listdir(CSRC_DIR) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(f for f in os.listdir(CSRC_DIR) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    for name in sources() + _headers():
        h.update(name.encode())
        with open(os.path.join(CSRC_DIR, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def _candidate_dirs() -> List[str]:
    dirs = []
    env = os.environ.get("SHARPI_BUILD_DIR")
    if env:
        dirs.append(env)
    dirs.append(os.path.join(CSRC_DIR, "_build"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"sharpi_build_{os.getuid()}"))
    return dirs


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def find_built() -> Optional[str]:
    """Path of an up-to-date library, or None."""
    want = source_hash()
    for d in _candidate_dirs():
        lib = os.path.join(d, LIB_NAME)
        stamp = os.path.join(d, "stamp.txt")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            try:
                with open(stamp) as f:
                    if f.read().strip() == want:
                        return lib
            except OSError:
                pass
    return None


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.isfile(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built (looked on PATH and in /opt/rocm/bin)")
    return exe


def _say(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[sharpi build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True, jobs: Optional[int] = None) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel build: tried " + ", ".join(_candidate_dirs()))
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 4)))
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir} ({jobs} at a time)", verbose)
    t0 = time.time()

    def compile_one(name: str) -> str:
        obj = os.path.join(out_dir, name[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC_DIR, name), "-o", obj]
        t = time.time()
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{p.stdout}")
        _say(f"  {name} done in {time.time() - t:.1f}s", verbose)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, srcs))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objs]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"link failed:\n{p.stdout}")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, "stamp.txt"), "w") as f:
        f.write(source_hash() + "\n")
    _say(f"built {lib} in {time.time() - t0:.1f}s", verbose)
    return lib


def ensure_built(verbose: bool = True) -> str:
    """The library's path; compiles it first if no up-to-date build exists."""
    lib = find_built()
    if lib is None:
        lib = build(verbose=verbose)
    return lib


if __name__ == "__main__":
    print(build())
