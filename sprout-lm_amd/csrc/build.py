"""Builds libsprout_hip.so from the HIP sources of this folder with hipcc, for gfx950."""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libsprout_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops is switched off: the compiler must not form packed float32 instructions.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-result"]
# Attention rescales its MFMA accumulators with vector instructions at every step; kept in AGPRs each
# such step would cost a move out and a move back, so these kernels take the VGPR form of MFMA.
FILE_FLAGS = {"attention_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources() -> list[str]:
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def source_digest() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(HERE)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(HERE, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()


def library_path(folder: str | None = None) -> str:
    return os.path.join(folder or HERE, LIB_NAME)


def is_current(folder: str | None = None) -> bool:
    lib, stamp = library_path(folder), library_path(folder) + ".digest"
    if not (os.path.exists(lib) and os.path.exists(stamp)):
        return False
    with open(stamp) as f:
        return f.read().strip() == source_digest()


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled (looked at $HIPCC, PATH, /opt/rocm/bin).")


def build(folder: str | None = None, verbose: bool = True, jobs: int | None = None) -> str:
    """Compile every source and link the library into `folder` (default: beside the sources)."""
    folder = folder or HERE
    hipcc = _hipcc()
    work = os.path.join(folder, "_build")
    os.makedirs(work, exist_ok=True)
    started = time.time()
    names = sources()

    def compile_one(name: str) -> str:
        obj = os.path.join(work, name[:-4] + ".o")
        cmd = [hipcc, *FLAGS, *FILE_FLAGS.get(name, []), "-c", os.path.join(HERE, name), "-o", obj]
        t0 = time.time()
        done = subprocess.run(cmd, capture_output=True, text=True)
        if done.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{done.stderr[-4000:]}")
        if verbose:
            print(f"[sprout build] compiled {name} in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
        return obj

    if verbose:
        print(f"[sprout build] compiling {len(names)} HIP sources for {ARCH} ...", file=sys.stderr, flush=True)
    done_compiling = threading.Event()

    def heartbeat() -> None:      # the largest source takes most of a minute: say that the build is alive
        while not done_compiling.wait(10.0):
            print(f"[sprout build] still compiling ({time.time() - started:.0f}s) ...", file=sys.stderr, flush=True)

    if verbose:
        threading.Thread(target=heartbeat, daemon=True).start()
    try:
        with ThreadPoolExecutor(max_workers=jobs or min(8, os.cpu_count() or 4)) as pool:
            objects = list(pool.map(compile_one, names))
    finally:
        done_compiling.set()
    tmp = library_path(folder) + f".tmp{os.getpid()}"
    done = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp, *objects],
                          capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"hipcc failed to link {LIB_NAME}:\n{done.stderr[-4000:]}")
    os.replace(tmp, library_path(folder))
    with open(library_path(folder) + ".digest", "w") as f:
        f.write(source_digest())
    if verbose:
        print(f"[sprout build] built {LIB_NAME} in {time.time() - started:.1f}s", file=sys.stderr, flush=True)
    return library_path(folder)


def ensure_built(verbose: bool = True) -> str:
    """Path of a library that matches the sources, building it at the first call.

    It is built beside the sources; where that folder cannot be written, in a
    per-user folder under the system's temporary directory.
    """
    if is_current():
        return library_path()
    if os.path.exists(library_path()) and os.environ.get("SPROUT_ALLOW_STALE_LIB") == "1":
        return library_path()
    try:
        probe = os.path.join(HERE, f".write_probe{os.getpid()}")
        open(probe, "w").close()
        os.remove(probe)
        return build(verbose=verbose)
    except OSError:
        folder = os.path.join(tempfile.gettempdir(), f"sprout_hip_{os.getuid()}_{source_digest()[:12]}")
        os.makedirs(folder, exist_ok=True)
        if is_current(folder):
            return library_path(folder)
        return build(folder, verbose=verbose)


if __name__ == "__main__":
    print(build())
