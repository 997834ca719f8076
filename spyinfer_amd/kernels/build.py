"""Builds and loads the HIP kernel library for gfx950.

The sources under ``spyinfer_amd/csrc`` are compiled with ``hipcc`` into one
shared library that is loaded with ctypes (no Python headers, so a build takes
seconds per file).  The library lies in ``csrc/_build``; if that folder cannot
be written, in a per-user folder under the system's temporary directory.
``load()`` builds only if no library matching the sources is there; ``build()``
always compiles.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libspyinfer_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc forms packed fp32 instructions on its own from float code otherwise
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-result", "-ffp-contract=fast"]

_lock = threading.Lock()
_lib = None


class KernelLibraryError(RuntimeError):
    pass


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".h", ".hpp")))


def source_digest() -> str:
    h = hashlib.sha256()
    for p in sources() + _headers():
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _candidate_dirs():
    dirs = [os.path.join(CSRC, "_build")]
    dirs.append(os.path.join(tempfile.gettempdir(), "spyinfer_amd_build_%d" % os.getuid()))
    return dirs


def _writable_dir():
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, ".probe_%d" % os.getpid())
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelLibraryError("no writable folder for the kernel library among: " + ", ".join(_candidate_dirs()))


def find_built():
    """Path of a built library that matches the current sources, or None."""
    digest = source_digest()
    for d in _candidate_dirs():
        lib = os.path.join(d, LIB_NAME)
        stamp = os.path.join(d, "digest.txt")
        if os.path.isfile(lib) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == digest:
                    return lib
    return None


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.isfile(exe):
        raise KernelLibraryError("hipcc not found: the HIP kernels cannot be compiled")
    return exe


def build(verbose: bool = True) -> str:
    """Compile every source for gfx950 and link the library.  Returns its path."""
    out_dir = _writable_dir()
    hipcc = _hipcc()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)          # hipcc wants a HOME for its temporary files
    env.setdefault("TMPDIR", tempfile.gettempdir())
    srcs = sources()
    objs = []
    t0 = time.time()
    procs = []
    for src in srcs:
        obj = os.path.join(out_dir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        cmd = [hipcc] + HIPCC_FLAGS + ["-I", CSRC, "-c", src, "-o", obj]
        procs.append((src, subprocess.Popen(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    for src, p in procs:
        if verbose:
            print("[spyinfer_amd] compiling %s for %s ..." % (os.path.basename(src), ARCH), file=sys.stderr, flush=True)
        while True:
            try:
                out, _ = p.communicate(timeout=20)
                break
            except subprocess.TimeoutExpired:
                if verbose:
                    print("[spyinfer_amd] ... still compiling (%.0f s)" % (time.time() - t0), file=sys.stderr, flush=True)
        if p.returncode != 0:
            for _, q in procs:
                if q.poll() is None:
                    q.kill()
            raise KernelLibraryError("hipcc failed on %s:\n%s" % (src, out.decode(errors="replace")))
    lib_tmp = os.path.join(out_dir, LIB_NAME + ".tmp%d" % os.getpid())
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o", lib_tmp] + objs
    r = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        raise KernelLibraryError("linking the kernel library failed:\n" + r.stdout.decode(errors="replace"))
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(lib_tmp, lib)
    with open(os.path.join(out_dir, "digest.txt"), "w") as f:
        f.write(source_digest())
    if verbose:
        print("[spyinfer_amd] kernel library built in %.0f s: %s" % (time.time() - t0, lib), file=sys.stderr, flush=True)
    return lib


def load() -> ctypes.CDLL:
    """The kernel library, built first if no matching one exists.  Raises if it cannot be had."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = find_built()
        if path is None:
            path = build(verbose=True)
        try:
            _lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError("cannot load the HIP kernel library %s: %s" % (path, e)) from None
        return _lib
