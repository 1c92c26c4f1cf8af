"""Compile the HIP sources of this folder and the C++ sources of ``host/`` into one shared library.

``build()`` compiles every ``*.hip`` file for gfx950 and every ``host/*.cpp`` file (plain C++: requests,
page pools, scheduler, step packing) with ``hipcc`` (objects in parallel, then one link) and
returns the path of ``libmini_engine_hip.so``. It prints a line per finished object, so a caller
that waits for a first-time build sees progress. No GPU is needed to compile.
"""

from __future__ import annotations

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libmini_engine_hip.so"
ARCH = "gfx950"
# Packed float32 instructions are switched off for every kernel of this library.
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# The GEMM library that plain products of prompts go to (csrc/gemm_library.hip calls it directly).
ROCM_LIB = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")
LINK_LIBS = [f"-L{ROCM_LIB}", f"-Wl,-rpath,{ROCM_LIB}", "-lhipblaslt"]


ROCM_INCLUDE = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include")
# The host sources are plain C++; those that launch kernels see the HIP runtime's C interface only.
HOST_FLAGS = ["-x", "c++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", ROCM_INCLUDE]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(HERE, "*.hip"))) + sorted(glob.glob(os.path.join(HERE, "host", "*.cpp")))


def default_lib_path() -> str:
    return os.path.join(HERE, LIB_NAME)


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP kernels cannot be compiled (looked at $HIPCC, PATH, /opt/rocm/bin)")


def is_current(lib_path: str) -> bool:
    if not os.path.exists(lib_path):
        return False
    t = os.path.getmtime(lib_path)
    deps = sources() + glob.glob(os.path.join(HERE, "*.h")) + glob.glob(os.path.join(HERE, "host", "*.h"))
    return all(os.path.getmtime(s) <= t for s in deps)


def _say(msg: str, quiet: bool) -> None:
    if not quiet:
        print(f"[mini-engine build] {msg}", file=sys.stderr, flush=True)


def build(out_dir: str | None = None, quiet: bool = False, jobs: int | None = None) -> str:
    """Compile everything and return the library path. ``out_dir`` defaults to this folder; when it
    is not writable a folder under the system's temporary directory is used instead."""
    hipcc = find_hipcc()
    out_dir = out_dir or HERE
    if not os.access(out_dir, os.W_OK):
        out_dir = os.path.join(tempfile.gettempdir(), f"mini_engine_hip_{os.getuid()}")
        os.makedirs(out_dir, exist_ok=True)
    os.makedirs(os.path.join(out_dir, "_build"), exist_ok=True)
    # objects of this build only: two processes that build at the same time do not share files
    obj_dir = tempfile.mkdtemp(prefix="objs_", dir=os.path.join(out_dir, "_build"))
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a home for its caches
    t0 = time.time()
    _say(f"compiling {len(srcs)} sources (HIP for {ARCH}, C++ host) with {jobs} jobs", quiet)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src).replace(".", "_") + ".o")
        flags = HOST_FLAGS if src.endswith(".cpp") else FLAGS
        cmd = [hipcc, *flags, "-I", HERE, "-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {os.path.basename(src)}:\n{r.stderr[-4000:]}")
        return obj

    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = {pool.submit(compile_one, s): s for s in srcs}
        for fut in concurrent.futures.as_completed(futures):
            objs.append(fut.result())
            _say(f"  {os.path.basename(futures[fut])} done ({len(objs)}/{len(srcs)}, {time.time() - t0:.0f}s)", quiet)
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *sorted(objs), *LINK_LIBS],
                       capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    shutil.rmtree(obj_dir, ignore_errors=True)
    _say(f"built {lib} in {time.time() - t0:.0f}s", quiet)
    return lib


if __name__ == "__main__":
    print(build())
