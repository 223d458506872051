"""Builds the native libraries: the gfx950 kernel library from the .hip sources in this folder
with hipcc, and the host library (cache bookkeeping, step metadata) from host/*.cpp with the host
compiler.

A library is kept beside the sources when that folder is writable (so a built tree can be
copied to a GPU machine), else in a per-user cache folder.  A stamp file records the hash of
the sources and flags it was built from; `ensure_built` rebuilds when they differ.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["elementwise.hip", "gemm.hip", "gemm_skinny.hip", "gemm_gate_up.hip", "attention.hip", "attention_mfma.hip", "attention_any.hip",
           "sampling.hip"]
HEADERS = ["api.h", "common.h"]
LIB_NAME = "libeasygpt_hip.so"
ARCH = "gfx950"
# packed-fp32 instructions are kept out of the generated code on purpose
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-pass-failed"]


HOST_SOURCES = ["host/cache_core.cpp"]
HOST_HEADERS = ["host/cache_core.h"]
HOST_LIB_NAME = "libeasygpt_host.so"
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra"]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str | None:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    return None


def source_hash() -> str:
    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:24]


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        with tempfile.NamedTemporaryFile(dir=d):
            pass
        return True
    except OSError:
        return False


def lib_dir() -> str:
    if _writable(HERE):
        return HERE
    base = os.environ.get("XDG_CACHE_HOME") or os.path.join(os.environ.get("HOME") or tempfile.gettempdir(), ".cache")
    d = os.path.join(base, "easy_gpt_cpp_amd")
    if _writable(d):
        return d
    d = os.path.join(tempfile.gettempdir(), f"easy_gpt_cpp_amd-{os.getuid()}")
    if _writable(d):
        return d
    raise BuildError("no writable folder for the kernel library")


def _paths():
    d = lib_dir()
    return os.path.join(d, LIB_NAME), os.path.join(d, "libeasygpt_hip.stamp")


def _log(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[easy_gpt.cpp_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every source for gfx950 and link the library.  Always compiles."""
    hipcc = _hipcc()
    if hipcc is None:
        raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")
    lib, stamp = _paths()
    obj_dir = tempfile.mkdtemp(prefix="egpt_build_")
    t0 = time.time()
    try:
        procs = []
        for src in SOURCES:
            obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
            cmd = [hipcc, *FLAGS, "-I", HERE, "-c", os.path.join(HERE, src), "-o", obj]
            _log(f"compiling {src} for {ARCH}", verbose)
            procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs = []
        for src, obj, p in procs:
            while True:
                try:
                    out, _ = p.communicate(timeout=20)
                    break
                except subprocess.TimeoutExpired:
                    _log(f"still compiling {src} ({time.time() - t0:.0f} s)", verbose)
            out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
            if p.returncode != 0:
                raise BuildError(f"hipcc failed on {src}:\n{out}")
            if out.strip():
                _log(out.strip(), verbose)
            objs.append(obj)
        tmp_lib = lib + f".tmp{os.getpid()}"
        cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp_lib]
        _log("linking " + os.path.basename(lib), verbose)
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise BuildError(f"link failed:\n{r.stdout}")
        os.replace(tmp_lib, lib)
        with open(stamp, "w") as f:
            f.write(source_hash())
        _log(f"built {lib} in {time.time() - t0:.1f} s", verbose)
        return lib
    finally:
        shutil.rmtree(obj_dir, ignore_errors=True)


def ensure_built(verbose: bool = True) -> str:
    """Path of a library that matches the sources; builds it if there is none."""
    lib, stamp = _paths()
    if os.path.isfile(lib) and os.path.isfile(stamp):
        with open(stamp) as f:
            if f.read().strip() == source_hash():
                return lib
        _log("kernel sources changed since the library was built; rebuilding", verbose)
    else:
        _log("no built kernel library found; building it (about a minute, once)", verbose)
    return build(verbose)


# ---------------------------------------------------------------------------------- the host library
def _host_compiler() -> str | None:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++"),
                 "/opt/rocm/llvm/bin/clang++"):
        if cand and (os.path.isfile(cand) or shutil.which(cand)):
            return cand
    return None


def host_source_hash() -> str:
    h = hashlib.sha256()
    for name in HOST_SOURCES + HOST_HEADERS:
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return h.hexdigest()[:24]


def _host_paths():
    d = lib_dir()
    return os.path.join(d, HOST_LIB_NAME), os.path.join(d, "libeasygpt_host.stamp")


def build_host(verbose: bool = True) -> str:
    """Compile the host library.  Always compiles."""
    cxx = _host_compiler()
    if cxx is None:
        raise BuildError("no C++ compiler found (looked at $CXX, g++, c++, clang++)")
    lib, stamp = _host_paths()
    tmp_lib = lib + f".tmp{os.getpid()}"
    t0 = time.time()
    cmd = [cxx, *HOST_FLAGS, "-I", os.path.join(HERE, "host"), *[os.path.join(HERE, s) for s in HOST_SOURCES], "-o", tmp_lib]
    _log("compiling " + ", ".join(HOST_SOURCES), verbose)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise BuildError(f"{cxx} failed:\n{r.stdout}")
    os.replace(tmp_lib, lib)
    with open(stamp, "w") as f:
        f.write(host_source_hash())
    _log(f"built {lib} in {time.time() - t0:.1f} s", verbose)
    return lib


def ensure_host_built(verbose: bool = True) -> str:
    lib, stamp = _host_paths()
    if os.path.isfile(lib) and os.path.isfile(stamp):
        with open(stamp) as f:
            if f.read().strip() == host_source_hash():
                return lib
    return build_host(verbose)


if __name__ == "__main__":
    print(build_host())
    print(build())
