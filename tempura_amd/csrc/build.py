"""Compile the HIP sources of this folder for gfx950 into one shared library.

The library is named after a hash of its sources and flags, so a changed source
never loads a stale build.  ``library_path()`` returns an existing build or
None; ``build()`` compiles (always), printing a progress line now and then;
``ensure_built()`` is what loaders call: use what is there, else build.

The build folder is ``_build`` beside the sources; when that is not writable
(a read-only checkout) a per-user folder under the system temp dir is used.
"""
from __future__ import annotations

import concurrent.futures
import glob
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
ARCH = "gfx950"
# -packed-fp32-ops is switched off: hipcc would otherwise form packed float32
# instructions from ordinary float code.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and $ROCM_PATH/bin): "
                       "the gfx950 kernels cannot be built")


def sources() -> List[str]:
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def _digest() -> str:
    h = hashlib.sha256()
    for p in sources() + sorted(glob.glob(os.path.join(HERE, "*.h"))):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def _build_dirs() -> List[str]:
    dirs = [os.path.join(HERE, "_build")]
    dirs.append(os.path.join(tempfile.gettempdir(), f"tempura_amd_build_{os.getuid()}"))
    return dirs


def _lib_name() -> str:
    return f"libtempura_hip_{_digest()}.so"


def library_path() -> Optional[str]:
    """Path of an existing build of the current sources, or None."""
    name = _lib_name()
    for d in _build_dirs():
        p = os.path.join(d, name)
        if os.path.exists(p):
            return p
    return None


def _writable_build_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w") as f:
                f.write("x")
            os.remove(probe)
            return d
        except OSError:
            continue
    raise RuntimeError("no writable folder for the kernel build: tried " + ", ".join(_build_dirs()))


def _run(cmd: List[str], what: str) -> None:
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{out}")
    if out.strip() and os.environ.get("TEMPURA_BUILD_VERBOSE"):
        print(out, file=sys.stderr)


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = _writable_build_dir()
    name = _lib_name()
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources in {HERE}")
    t0 = time.time()
    done = threading.Event()

    def say(msg: str) -> None:
        if verbose:
            print(f"[tempura_amd] {msg}", file=sys.stderr, flush=True)

    def ticker() -> None:
        while not done.wait(10.0):
            say(f"still compiling kernels for {ARCH} ... {time.time() - t0:.0f} s")

    say(f"compiling {len(srcs)} kernel sources for {ARCH} with {hipcc}")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    tag = f"{os.getpid()}"
    objs = [os.path.join(out_dir, os.path.basename(s)[:-4] + f".{tag}.o") for s in srcs]
    try:
        workers = max(1, min(len(srcs), os.cpu_count() or 1, 16))
        with concurrent.futures.ThreadPoolExecutor(workers) as ex:
            futs = [ex.submit(_run, [hipcc, *FLAGS, "-c", s, "-o", o], f"compiling {os.path.basename(s)}")
                    for s, o in zip(srcs, objs)]
            for f in futs:
                f.result()
        tmp = os.path.join(out_dir, name + f".{tag}.tmp")
        _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp], "linking")
        # A kernel whose host stub was not emitted links all the same and fails when the library is loaded: load it
        # here (in a process of its own; loading needs no GPU), so that a build says so and not the first user.
        check = subprocess.run([sys.executable, "-c", "import ctypes, sys; ctypes.CDLL(sys.argv[1])", tmp],
                               capture_output=True, text=True)
        if check.returncode != 0:
            os.remove(tmp)
            raise RuntimeError("the kernel library was linked but does not load:\n" + check.stderr.strip()[-2000:])
        final = os.path.join(out_dir, name)
        os.replace(tmp, final)
    finally:
        done.set()
        for o in objs:
            if os.path.exists(o):
                os.remove(o)
    for old in glob.glob(os.path.join(out_dir, "libtempura_hip_*.so")):
        if os.path.basename(old) != name:
            try:
                os.remove(old)
            except OSError:
                pass
    say(f"kernels built in {time.time() - t0:.0f} s: {final}")
    return final


def ensure_built(verbose: bool = True) -> str:
    return library_path() or build(verbose)


# ---- the host library: plain C++ (no GPU code), needed on machines without a GPU too ------------
# (no contraction into fused multiply-adds: counter_normal.h must round as the device kernel does)
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-pthread", "-ffp-contract=off"]


def host_sources() -> List[str]:
    return sorted(glob.glob(os.path.join(HERE, "host", "*.cpp")))


def _host_lib_name() -> str:
    h = hashlib.sha256()
    for p in host_sources() + [os.path.join(HERE, "counter_normal.h")]:
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HOST_FLAGS).encode())
    return f"libtempura_host_{h.hexdigest()[:16]}.so"


def host_library_path() -> Optional[str]:
    name = _host_lib_name()
    for d in _build_dirs():
        p = os.path.join(d, name)
        if os.path.exists(p):
            return p
    return None


def build_host(verbose: bool = True) -> str:
    """Compile the host library (always); returns its path."""
    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++") or shutil.which("clang++")
    if not cxx:
        raise RuntimeError("no C++ compiler found (looked at $CXX, g++, c++, clang++): the host library cannot be built")
    out_dir = _writable_build_dir()
    name = _host_lib_name()
    t0 = time.time()
    tmp = os.path.join(out_dir, name + f".{os.getpid()}.tmp")
    _run([cxx, *HOST_FLAGS, *host_sources(), "-o", tmp], "compiling the host library")
    final = os.path.join(out_dir, name)
    os.replace(tmp, final)
    for old in glob.glob(os.path.join(out_dir, "libtempura_host_*.so")):
        if os.path.basename(old) != name:
            try:
                os.remove(old)
            except OSError:
                pass
    if verbose:
        print(f"[tempura_amd] host library built in {time.time() - t0:.0f} s: {final}", file=sys.stderr, flush=True)
    return final


def ensure_host_built(verbose: bool = True) -> str:
    return host_library_path() or build_host(verbose)


if __name__ == "__main__":
    print(build_host())
    print(build())
