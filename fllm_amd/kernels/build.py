"""Compiles the HIP sources under csrc/ into one shared library for gfx950.

The library is built in-tree (next to this file) when the folder can be written, otherwise under
the temporary folder.  Each source is compiled by its own hipcc process; a line is printed when a
source starts and when it ends, so a first call that has to compile says what it is doing.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor, as_completed
from typing import List, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
LIB_NAME = "libfllm_kernels.so"
ARCH = "gfx950"
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
# flags of single sources: the random-weights generator must round every product and every sum on its own
SOURCE_FLAGS = {"random_fill.hip": ["-ffp-contract=off"]}


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith(".hip"))


def _source_digest() -> str:
    h = hashlib.sha256()
    for path in sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith((".hip", ".h"))):
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    h.update(repr(sorted(SOURCE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the kernel library cannot be built (looked at $HIPCC, PATH, /opt/rocm/bin)")


def in_tree_library() -> str:
    return os.path.join(_HERE, LIB_NAME)


def _fallback_dir() -> str:
    return os.path.join(tempfile.gettempdir(), f"fllm_amd_build_{os.getuid()}_{_source_digest()}")


def _stamp_matches(lib: str) -> bool:
    """True when `lib` exists and the digest written beside it at build time is that of the present sources."""
    stamp = lib + ".digest"
    if not (os.path.isfile(lib) and os.path.isfile(stamp)):
        return False
    with open(stamp) as fh:
        return fh.read().strip() == _source_digest()


def find_library() -> Optional[str]:
    """A library built from the present sources: the in-tree one, else the one under the temporary folder (whose
    folder name carries the digest too).  A library without a digest beside it, or with another one, is stale:
    None is returned and the caller builds."""
    for lib in (in_tree_library(), os.path.join(_fallback_dir(), LIB_NAME)):
        if _stamp_matches(lib):
            return lib
    return None


def _log(msg: str, quiet: bool) -> None:
    if not quiet:
        print(f"[fllm_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = False, quiet: bool = False, jobs: Optional[int] = None) -> str:
    """Builds the library (unless one that matches the sources exists and `force` is false) and
    returns its path."""
    if not force:
        existing = find_library()
        if existing:
            return existing
    hipcc = _hipcc()
    out_dir = _HERE
    try:
        probe = os.path.join(out_dir, f".write_probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
    except OSError:
        out_dir = _fallback_dir()
        os.makedirs(out_dir, exist_ok=True)
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    t0 = time.time()
    _log(f"compiling {len(srcs)} HIP sources for {ARCH} with {jobs} jobs into {out_dir}", quiet)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        started = time.time()
        proc = subprocess.run([hipcc, *HIPCC_FLAGS, *SOURCE_FLAGS.get(os.path.basename(src), []), "-I", CSRC, "-c", src, "-o", obj],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}")
        _log(f"  {os.path.basename(src)} done in {time.time() - started:.1f}s", quiet)
        return obj

    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(compile_one, s) for s in srcs]
        for fut in as_completed(futures):
            objs.append(fut.result())
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    proc = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp, *sorted(objs)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {lib}:\n{proc.stdout}")
    os.replace(tmp, lib)
    with open(lib + ".digest", "w") as fh:
        fh.write(_source_digest())
    _log(f"built {lib} in {time.time() - t0:.1f}s", quiet)
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
