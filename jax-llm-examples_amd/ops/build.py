"""Compiles the HIP sources under ``csrc/`` into one shared library for gfx950.

The library's file name carries a hash of the sources and flags, so a stale
build is never loaded.  ``library_path()`` returns the built library, compiling
it first if it is not there (each source in its own ``hipcc`` process, a
progress line every few seconds).  The build folder is ``csrc/_build`` inside
the package if that is writable, else a per-user folder under the system's
temporary directory.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no packed float32 math
    "-Wno-unused-command-line-argument",
]


def sources() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    for name in sources() + _headers():
        h.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled (set HIPCC or install ROCm)")


def _build_dir() -> str:
    for cand in (os.environ.get("JLE_BUILD_DIR"), os.path.join(CSRC, "_build"),
                 os.path.join(tempfile.gettempdir(), f"jle-build-{os.getuid()}")):
        if not cand:
            continue
        try:
            os.makedirs(cand, exist_ok=True)
            probe = os.path.join(cand, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return cand
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel build")


def _say(msg: str) -> None:
    print(f"[jle build] {msg}", file=sys.stderr, flush=True)


def find_library() -> str | None:
    name = f"libjle-{source_hash()}.so"
    for d in (os.environ.get("JLE_BUILD_DIR"), os.path.join(CSRC, "_build"),
              os.path.join(tempfile.gettempdir(), f"jle-build-{os.getuid()}")):
        if d and os.path.exists(os.path.join(d, name)):
            return os.path.join(d, name)
    return None


def build(force: bool = False, jobs: int | None = None) -> str:
    if not force:
        found = find_library()
        if found:
            return found
    hipcc = _hipcc()
    out_dir = _build_dir()
    tag = source_hash()
    obj_dir = os.path.join(out_dir, f"obj-{tag}-{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 4)))
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} with {jobs} jobs (first use; this takes a minute or two)")
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc, *FLAGS, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        return obj

    objs = []
    with concurrent.futures.ThreadPoolExecutor(jobs) as pool:
        futs = {pool.submit(compile_one, s): s for s in srcs}
        pending = set(futs)
        while pending:
            done, pending = concurrent.futures.wait(pending, timeout=10)
            for f in done:
                objs.append(f.result())
            _say(f"{len(srcs) - len(pending)}/{len(srcs)} sources compiled after {time.time() - t0:.0f} s")
    lib = os.path.join(out_dir, f"libjle-{tag}.so")
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *sorted(objs), "-o", tmp],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"linking the kernel library failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, lib)
    shutil.rmtree(obj_dir, ignore_errors=True)
    for f in os.listdir(out_dir):  # older builds
        if f.startswith("libjle-") and f.endswith(".so") and f != os.path.basename(lib):
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def library_path() -> str:
    return build(force=False)
