"""Building and finding the HIP kernel library (``libtli_kernels.so``).

The sources under ``csrc/`` are compiled for gfx950 with hipcc, each file on
its own, in parallel, and linked into one shared library beside them.  A
library already built is used as it is unless a source is newer.  If the
package folder cannot be written (an installed, read-only copy) the library is
built in a per-user folder under the system's temporary directory.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libtli_kernels.so"
ARCH = "gfx950"
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
         # packed float32 instructions are switched off for all device code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # MFMA accumulators stay in ordinary vector registers: the softmax rescales them
         # with vector instructions, and copies to and from the accumulation registers
         # cost more than the registers they save
         "-mllvm", "-amdgpu-mfma-vgpr-form=1",
         "-Wno-unused-command-line-argument"]


class BuildError(RuntimeError):
    pass


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _writable(folder: str) -> bool:
    try:
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _fallback_dir() -> str:
    tag = hashlib.sha1(CSRC.encode()).hexdigest()[:10]
    folder = os.path.join(tempfile.gettempdir(), f"tli-kernels-{os.getuid()}-{tag}")
    os.makedirs(folder, exist_ok=True)
    return folder


def candidates() -> List[str]:
    return [os.path.join(CSRC, LIB_NAME), os.path.join(_fallback_dir(), LIB_NAME)]


def _fresh(lib: str) -> bool:
    if not os.path.exists(lib):
        return False
    built = os.path.getmtime(lib)
    return all(os.path.getmtime(s) <= built for s in sources() + _headers())


def find_library() -> Optional[str]:
    for lib in candidates():
        if _fresh(lib):
            return lib
    return None


def build_library(force: bool = False, verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    if not force:
        lib = find_library()
        if lib:
            return lib
    out_dir = CSRC if _writable(CSRC) else _fallback_dir()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    hipcc = _hipcc()
    srcs = sources()
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[tli build] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *FLAGS, "-c", src, "-o", obj]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                              env={**os.environ, "HOME": os.environ.get("HOME") or out_dir})
        return src, obj, proc.returncode, proc.stdout

    objs = []
    jobs = min(8, len(srcs), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(compile_one, s) for s in srcs]
        for n, fut in enumerate(as_completed(futures), 1):
            src, obj, code, text = fut.result()
            if code != 0:
                raise BuildError(f"hipcc failed on {src}:\n{text}")
            objs.append(obj)
            say(f"  {n}/{len(srcs)} {os.path.basename(src)} ({time.time() - t0:.0f} s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    proc = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *sorted(objs),
                           "-o", tmp], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          env={**os.environ, "HOME": os.environ.get("HOME") or out_dir})
    if proc.returncode != 0:
        raise BuildError(f"linking {lib} failed:\n{proc.stdout}")
    os.replace(tmp, lib)
    say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


# ---- the C ABI of the engine (capi/): host code only, a Python interpreter embedded ----------
CAPI = os.path.join(os.path.dirname(CSRC), "capi")
ENGINE_LIB = "libtli_engine.so"


def find_engine_api() -> Optional[str]:
    lib = os.path.join(CAPI, ENGINE_LIB)
    srcs = [os.path.join(CAPI, f) for f in ("tli_engine.cpp", "tli_engine.h")]
    if os.path.exists(lib) and all(os.path.getmtime(s) <= os.path.getmtime(lib) for s in srcs):
        return lib
    return None


def build_engine_api(force: bool = False, verbose: bool = True) -> str:
    """Compile ``capi/tli_engine.cpp`` (the engine for C and C++ programs) against this
    interpreter's headers and library; returns the path of ``libtli_engine.so``."""
    import sysconfig
    if not force:
        lib = find_engine_api()
        if lib:
            return lib
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if not cxx:
        raise BuildError("no C++ compiler was found for the engine's C ABI (g++, c++ or clang++)")
    include = sysconfig.get_paths()["include"]
    libdir = sysconfig.get_config_var("LIBDIR") or ""
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_python_version()
    lib = os.path.join(CAPI, ENGINE_LIB)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [cxx, "-O2", "-std=c++17", "-shared", "-fPIC", f"-I{include}", os.path.join(CAPI, "tli_engine.cpp"),
           "-o", tmp, f"-L{libdir}", f"-lpython{version}", "-ldl", f"-Wl,-rpath,{libdir}"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise BuildError(f"building {lib} failed:\n{proc.stdout}")
    os.replace(tmp, lib)
    if verbose:
        print(f"[tli build] built {lib}", file=sys.stderr, flush=True)
    return lib


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv))
    print(build_engine_api(force="--force" in sys.argv))
