"""Compiles the HIP sources of this folder into one shared library for gfx950.

`build(force=True)` always compiles (the "does it build" check).  `ensure_built()`
compiles only when no library is there or a source is newer; tests, the bench and the
command line call that.  The library lies beside the sources; when that folder cannot
be written (a read-only checkout), it goes to a per-user folder under the system's
temporary directory instead.

Flags: -O3, gfx950 only, and packed 32-bit float instructions switched off (some of
their forms have given wrong results on this hardware).
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "librbitnet_hip.so"
ARCH = "gfx950"
SOURCES = ["elementwise.hip", "gemm_generic.hip", "gemm_mfma.hip", "gemm_skinny.hip", "gemm_tiled.hip",
           "attention_generic.hip", "attention_mfma.hip", "sampling.hip", "weights_init.hip", "probe.hip", "plan.hip"]
HEADERS = ["api.h", "tune.h", "common.h", "mfma.h", "gemm_internal.h"]
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-result", "-Wno-unknown-warning-option"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


def _source_digest() -> str:
    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
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


def _candidate_dirs() -> List[str]:
    fallback = os.path.join(tempfile.gettempdir(), f"rbitnet_amd_build_{os.getuid()}")
    return [HERE, fallback]


def library_path() -> Optional[str]:
    """The newest built library that matches the sources, if any."""
    digest = _source_digest()
    for folder in _candidate_dirs():
        lib = os.path.join(folder, LIB_NAME)
        stamp = lib + ".stamp"
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == digest:
                    return lib
    return None


def any_library_path() -> Optional[str]:
    """A built library whatever its stamp says (for a tree whose sources cannot be read)."""
    for folder in _candidate_dirs():
        lib = os.path.join(folder, LIB_NAME)
        if os.path.isfile(lib):
            return lib
    return None


def _progress(stop: threading.Event, what: str, t0: float) -> None:
    while not stop.wait(15.0):
        print(f"[rbitnet_amd] still compiling {what} ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)


def build(force: bool = True, verbose: bool = True) -> str:
    """Compile every source with hipcc and link the library.  Returns its path."""
    if not force:
        lib = library_path()
        if lib:
            return lib
    hipcc = _hipcc()
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the built kernel library")
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    t0 = time.time()
    if verbose:
        print(f"[rbitnet_amd] compiling {len(SOURCES)} HIP sources for {ARCH} into {out_dir}",
              file=sys.stderr, flush=True)
    stop = threading.Event()
    ticker = threading.Thread(target=_progress, args=(stop, "the HIP kernels", t0), daemon=True)
    if verbose:
        ticker.start()
    try:
        procs = []
        objs = []
        for src in SOURCES:
            obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
            objs.append(obj)
            cmd = [hipcc] + FLAGS + ["-c", os.path.join(HERE, src), "-o", obj]
            procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
        for src, p in procs:
            out, err = p.communicate()
            if p.returncode != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n{err[-4000:]}")
        lib = os.path.join(out_dir, LIB_NAME)
        tmp = lib + f".tmp{os.getpid()}"
        cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp] + objs
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"linking {LIB_NAME} failed:\n{r.stderr[-4000:]}")
        os.replace(tmp, lib)
        with open(lib + ".stamp", "w") as f:
            f.write(_source_digest())
    finally:
        stop.set()
    if verbose:
        print(f"[rbitnet_amd] built {lib} in {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    return lib


def ensure_built(verbose: bool = True) -> str:
    lib = library_path()
    if lib:
        return lib
    try:
        return build(force=True, verbose=verbose)
    except RuntimeError:
        stale = any_library_path()
        if stale:
            print(f"[rbitnet_amd] warning: could not rebuild, using existing {stale}", file=sys.stderr, flush=True)
            return stale
        raise


# ---------------------------------------------------------------- the plain C++ twins (no GPU)
PLAIN_LIB_NAME = "librbitnet_plain.so"
PLAIN_SELFTEST_NAME = "plain_selftest"
PLAIN_SOURCES = ["plain.cpp", "plain.h", "plain_selftest.cpp"]
PLAIN_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Werror"]
SANITIZE = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-static-libasan",
            "-static-libubsan", "-g"]


def _host_compiler() -> str:
    for cand in (os.environ.get("CXX"), shutil.which("g++"), shutil.which("c++"), shutil.which("clang++")):
        if cand and os.path.isfile(cand):
            return cand
    raise RuntimeError("no host C++ compiler found (looked at $CXX, g++, c++, clang++)")


def _plain_digest() -> str:
    h = hashlib.sha256()
    for name in PLAIN_SOURCES:
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(PLAIN_FLAGS + SANITIZE).encode())
    return h.hexdigest()[:16]


def _plain_built(name: str) -> Optional[str]:
    digest = _plain_digest()
    for folder in _candidate_dirs():
        path = os.path.join(folder, name)
        if os.path.isfile(path) and os.path.isfile(path + ".stamp"):
            with open(path + ".stamp") as f:
                if f.read().strip() == digest:
                    return path
    return None


def _compile_host(args: List[str], out_name: str) -> str:
    out_dir = next((d for d in _candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("no writable folder for the built twins")
    out = os.path.join(out_dir, out_name)
    tmp = out + f".tmp{os.getpid()}"
    r = subprocess.run([_host_compiler()] + args + ["-o", tmp], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"compiling {out_name} failed:\n{r.stderr[-4000:]}")
    os.replace(tmp, out)
    with open(out + ".stamp", "w") as f:
        f.write(_plain_digest())
    return out


def build_plain(force: bool = False) -> str:
    """The twins as a shared library for ctypes (host compiler, no GPU code).  Returns its path."""
    if not force:
        lib = _plain_built(PLAIN_LIB_NAME)
        if lib:
            return lib
    return _compile_host(PLAIN_FLAGS + ["-shared", os.path.join(HERE, "plain.cpp")], PLAIN_LIB_NAME)


def build_plain_selftest(force: bool = False) -> str:
    """The twins and their self-test as one program under the address and undefined-behaviour
    sanitizers (their run-time parts linked in statically, so that nothing has to be preloaded)."""
    if not force:
        exe = _plain_built(PLAIN_SELFTEST_NAME)
        if exe:
            return exe
    return _compile_host(PLAIN_FLAGS + SANITIZE + [os.path.join(HERE, "plain.cpp"), os.path.join(HERE, "plain_selftest.cpp")],
                         PLAIN_SELFTEST_NAME)


if __name__ == "__main__":
    print(build(force=True))
    print(build_plain(force=True))
    print(build_plain_selftest(force=True))
