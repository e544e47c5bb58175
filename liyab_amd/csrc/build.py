"""Builds the HIP kernels into one shared library for gfx950.

`build()` compiles every `.hip` file beside this script with hipcc, in
parallel, and links `liyab_amd/_lib/libliyab_hip.so`; it prints a line per
file so that a first call in a fresh checkout shows progress. When the
package folder cannot be written to, the library goes to a per-user folder
under the system's temporary directory instead. Nothing here needs a GPU:
hipcc cross-compiles. `build_host()` does the same for the host-side C++
under `host/` (the cache manager's bookkeeping and a step's metadata), with
the system's C++ compiler, into `libliyab_host.so`; that library has nothing
to do with HIP and loads on a machine without a GPU.
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

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
LIB_NAME = "libliyab_hip.so"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed 32-bit float instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# Matrix-instruction results in ordinary vector registers for kernels that work on them with
# vector instructions between the products (softmax on the scores, rescaling of the outputs):
# by default they land in accumulation registers and every such use costs a move each way.
VGPR_MFMA = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
FILE_FLAGS = {
    "attention_prefill.hip": VGPR_MFMA,
}


def sources() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def headers() -> List[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    for p in sources() + headers():
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    h.update(repr(sorted(FILE_FLAGS.items())).encode())
    return h.hexdigest()[:16]


def hipcc_path() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs() -> List[str]:
    """Where the library may live, in the order they are tried."""
    user = f"liyab_amd_{os.getuid()}_{source_hash()}"
    return [os.path.join(PKG, "_lib"), os.path.join(tempfile.gettempdir(), user)]


def find_library() -> Optional[str]:
    for d in lib_dirs():
        p = os.path.join(d, LIB_NAME)
        if os.path.isfile(p):
            return p
    return None


def is_stale(lib_path: str) -> bool:
    try:
        with open(lib_path + ".hash") as f:
            return f.read().strip() != source_hash()
    except OSError:
        return True


def _say(msg: str, quiet: bool) -> None:
    if not quiet:
        print(f"[liyab_amd build] {msg}", file=sys.stderr, flush=True)


def build(quiet: bool = False, jobs: Optional[int] = None) -> str:
    """Compiles and links; returns the library's path."""
    hipcc = hipcc_path()
    if hipcc is None:
        raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")
    out_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the kernel library: tried " + ", ".join(lib_dirs()))
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = out_dir  # the compiler driver wants some home folder
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 1)))
    t0 = time.time()
    _say(f"compiling {len(srcs)} HIP files for {ARCH} with {jobs} jobs into {out_dir}", quiet)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        t = time.time()
        extra = FILE_FLAGS.get(os.path.basename(src), [])
        r = subprocess.run([hipcc, *FLAGS, *extra, "-I", CSRC, "-c", src, "-o", obj], env=env, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {os.path.basename(src)}:\n{r.stdout}\n{r.stderr}")
        _say(f"  {os.path.basename(src)} done in {time.time() - t:.0f} s", quiet)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, srcs))
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], env=env,
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(source_hash())
    shutil.rmtree(obj_dir, ignore_errors=True)
    _say(f"built {lib} in {time.time() - t0:.0f} s", quiet)
    return lib


# -- the host library ------------------------------------------------------------------
HOST_DIR = os.path.join(CSRC, "host")
HOST_LIB_NAME = "libliyab_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra"]


def host_sources() -> List[str]:
    return sorted(os.path.join(HOST_DIR, f) for f in os.listdir(HOST_DIR) if f.endswith(".cpp"))


def host_hash() -> str:
    h = hashlib.sha256()
    for f in sorted(os.listdir(HOST_DIR)):
        if f.endswith((".cpp", ".h")):
            h.update(f.encode())
            with open(os.path.join(HOST_DIR, f), "rb") as fh:
                h.update(fh.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()[:16]


def host_lib_dirs() -> List[str]:
    return [os.path.join(PKG, "_lib"), os.path.join(tempfile.gettempdir(), f"liyab_amd_{os.getuid()}_host_{host_hash()}")]


def find_host_library() -> Optional[str]:
    """The host library built from the current sources, if there is one."""
    for d in host_lib_dirs():
        p = os.path.join(d, HOST_LIB_NAME)
        try:
            with open(p + ".hash") as f:
                if f.read().strip() == host_hash() and os.path.isfile(p):
                    return p
        except OSError:
            pass
    return None


def cxx_path() -> Optional[str]:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"), hipcc_path()):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def build_host(quiet: bool = False) -> str:
    cxx = cxx_path()
    if cxx is None:
        raise RuntimeError("no C++ compiler was found (looked at $CXX, g++, c++, clang++, hipcc): the host library cannot be built")
    out_dir = next((d for d in host_lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the host library: tried " + ", ".join(host_lib_dirs()))
    t0 = time.time()
    lib = os.path.join(out_dir, HOST_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    r = subprocess.run([cxx, *HOST_FLAGS, "-I", HOST_DIR, "-o", tmp, *host_sources()], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building {HOST_LIB_NAME} failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, lib)
    with open(lib + ".hash", "w") as f:
        f.write(host_hash())
    _say(f"built {lib} in {time.time() - t0:.0f} s", quiet)
    return lib


# -- the C library over the engine --------------------------------------------------------
CAPI_DIR = os.path.join(CSRC, "capi")
CAPI_LIB_NAME = "libliyab_engine.so"


def build_engine_capi(quiet: bool = False) -> str:
    """Builds `capi/liyab_engine_c.cpp` (the engine for C programs: it runs `liyab_amd` in a Python
    interpreter inside the caller's process) into `_lib/libliyab_engine.so`, linked against this
    interpreter's library. Returns its path."""
    import sysconfig

    cxx = cxx_path()
    if cxx is None:
        raise RuntimeError("no C++ compiler was found (looked at $CXX, g++, c++, clang++, hipcc)")
    out_dir = next((d for d in host_lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the engine's C library: tried " + ", ".join(host_lib_dirs()))
    include = sysconfig.get_config_var("INCLUDEPY")
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_config_var("VERSION")
    libdirs = [d for d in (sysconfig.get_config_var("LIBDIR"), sysconfig.get_config_var("LIBPL")) if d]
    lib = os.path.join(out_dir, CAPI_LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-I", include, "-I", CAPI_DIR, "-o", tmp,
           os.path.join(CAPI_DIR, "liyab_engine_c.cpp"), *[f"-L{d}" for d in libdirs], f"-lpython{version}", "-ldl",
           *[f"-Wl,-rpath,{d}" for d in libdirs]]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building {CAPI_LIB_NAME} failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, lib)
    _say(f"built {lib}", quiet)
    return lib


def build_host_selftest(sanitize: bool = True, out_dir: Optional[str] = None) -> str:
    """Compiles `host/selftest/selftest.cpp` with the host sources into an executable of its own
    and returns its path. `sanitize`: with the address and undefined-behaviour sanitizers
    (-fsanitize=address,undefined, no recovery: the first finding ends the run). The executable
    links nothing of Python or HIP, so the sanitizers' runtime is the only thing loaded with it."""
    cxx = cxx_path()
    if cxx is None:
        raise RuntimeError("no C++ compiler was found (looked at $CXX, g++, c++, clang++, hipcc)")
    out_dir = out_dir or tempfile.mkdtemp(prefix="liyab_host_selftest_")
    exe = os.path.join(out_dir, "host_selftest_san" if sanitize else "host_selftest")
    flags = ["-O1", "-g", "-std=c++17", "-Wall", "-Wextra"]
    if sanitize:
        # the sanitizers' runtime linked in, so that it need not come first among preloaded libraries
        flags += ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer",
                  "-static-libasan", "-static-libubsan"]
    srcs = [p for p in host_sources() if not p.endswith("c_api.cpp")] + [os.path.join(HOST_DIR, "selftest", "selftest.cpp")]
    r = subprocess.run([cxx, *flags, "-I", HOST_DIR, "-o", exe, *srcs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"building the host self-test failed:\n{r.stdout}\n{r.stderr}")
    return exe


if __name__ == "__main__":
    print(build_host())
    print(build())
