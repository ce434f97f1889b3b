"""Compiling the gfx950 kernels into one shared library with hipcc, and finding that library.

``build()`` compiles every ``*.hip`` of this folder (in parallel, one hipcc per file) and links
``liblucciola_hip.so`` next to the sources; ``library_path()`` returns the built library and
builds it first if it is missing or older than the sources.  Progress goes to stderr, one
line per file, so that a first call that has to compile does not look hung.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import FIRST_COMPLETED, ThreadPoolExecutor, wait
from typing import List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "liblucciola_hip.so"
ARCH = "gfx950"
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    "-fvisibility=hidden", "-fno-gpu-rdc",
    # packed float32 instructions are switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the kernels keep accumulators and operands in register arrays that only fully unrolled
    # loops can index; no size estimate may stop an unroll that the source asks for
    "-mllvm", "-pragma-unroll-threshold=1000000",
]


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[lucciola_amd build] {msg}", file=sys.stderr, flush=True)


def sources() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for name in _headers() + sources():
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def find_hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _out_dir() -> str:
    """Next to the sources when that folder can be written, else a per-user temporary folder."""
    if os.access(HERE, os.W_OK):
        return HERE
    d = os.path.join(tempfile.gettempdir(), f"lucciola_amd_build_{os.getuid()}")
    os.makedirs(d, exist_ok=True)
    return d


def _candidates() -> List[str]:
    dirs = [HERE, os.path.join(tempfile.gettempdir(), f"lucciola_amd_build_{os.getuid()}")]
    return [os.path.join(d, LIB_NAME) for d in dirs]


def _is_current(lib: str) -> bool:
    stamp = lib + ".hash"
    if not (os.path.isfile(lib) and os.path.isfile(stamp)):
        return False
    with open(stamp, "r") as fh:
        return fh.read().strip() == source_hash()


def build(force: bool = True, jobs: Optional[int] = None) -> str:
    """Compile and link; returns the library's path."""
    hipcc = find_hipcc()
    if hipcc is None:
        raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the gfx950 "
                         "kernels cannot be compiled")
    out_dir = _out_dir()
    lib = os.path.join(out_dir, LIB_NAME)
    if not force and _is_current(lib):
        return lib
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 1)))
    _log(f"compiling {len(srcs)} kernel files for {ARCH} with {jobs} jobs ...")
    t0 = time.time()

    def compile_one(name: str) -> str:
        obj = os.path.join(obj_dir, name[:-4] + ".o")
        cmd = [hipcc] + FLAGS + ["-I", HERE, "-c", os.path.join(HERE, name), "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise BuildError(f"hipcc failed on {name}:\n{proc.stdout}")
        return obj

    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = {pool.submit(compile_one, s): s for s in srcs}
        pending = set(futures)
        while pending:
            # a line every ten seconds at the least: the largest file takes half a minute
            done, pending = wait(pending, timeout=10, return_when=FIRST_COMPLETED)
            for fut in done:
                objs.append(fut.result())
                _log(f"  {futures[fut]} done ({time.time() - t0:.0f} s)")
            if not done:
                _log(f"  still compiling {', '.join(sorted(futures[f] for f in pending))} ({time.time() - t0:.0f} s)")
    tmp_lib = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-o", tmp_lib] + sorted(objs)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"linking {LIB_NAME} failed:\n{proc.stdout}")
    os.replace(tmp_lib, lib)
    with open(lib + ".hash", "w") as fh:
        fh.write(source_hash())
    _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def library_path(build_if_needed: bool = True) -> str:
    """The built library; compiled now if there is none that matches the sources."""
    for lib in _candidates():
        if _is_current(lib):
            return lib
    if not build_if_needed:
        raise BuildError(f"{LIB_NAME} is not built (run `python -c 'import __graft_entry__ as g; "
                         f"g.build()'` or lucciola_amd.csrc.build.build())")
    return build(force=True)


if __name__ == "__main__":
    print(build(force=True))
