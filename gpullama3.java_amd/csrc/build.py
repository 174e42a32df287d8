"""Compiles the HIP sources of this folder for gfx950 into one shared library.

The library's file name carries a hash of the sources and flags, so a library
that does not match the sources is never loaded. It is built in-tree
(``csrc/_built``), or under the temporary folder when the tree is read-only.
"""
from __future__ import annotations

import glob
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
# (kernarg preload: a kernel's first arguments arrive in scalar registers with the dispatch, where a kernel would
# otherwise begin with a trip to memory for them)
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-mllvm", "-amdgpu-kernarg-preload-count=16"]
_NOISE = "is not a recognized feature for this target"


def sources():
    return sorted(glob.glob(os.path.join(HERE, "*.hip")))


def headers():
    return sorted(glob.glob(os.path.join(HERE, "*.h")))


def source_hash():
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for p in sources() + headers():
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def _hipcc():
    for c in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.exists(c):
            return c
    raise RuntimeError("hipcc not found: the HIP kernels cannot be built (is ROCm installed under /opt/rocm?)")


def _out_dirs():
    yield os.path.join(HERE, "_built")
    yield os.path.join(tempfile.gettempdir(), f"gl3hip-{os.getuid()}")


def library_path(must_exist=True):
    """Path of the built library for the current sources, or None."""
    name = f"gl3hip-{source_hash()}.so"
    for d in _out_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def _say(msg):
    print(f"[gpullama3.java_amd build] {msg}", file=sys.stderr, flush=True)


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if _NOISE not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def build(force=False, verbose=True):
    """Compile if needed (always when ``force``) and return the library's path."""
    if not force:
        p = library_path()
        if p:
            return p
    hipcc = _hipcc()
    name = f"gl3hip-{source_hash()}.so"
    last_error = None
    for d in _out_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".w{os.getpid()}")
            open(probe, "w").close()
            os.remove(probe)
        except OSError as e:
            last_error = e
            continue
        work = tempfile.mkdtemp(prefix="obj-", dir=d)
        try:
            srcs = sources()
            t0 = time.time()
            if verbose:
                _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {d}")

            def one(src):
                obj = os.path.join(work, os.path.basename(src) + ".o")
                t = time.time()
                out = _run([hipcc, *FLAGS, "-I", HERE, "-c", src, "-o", obj])
                if verbose:
                    _say(f"  {os.path.basename(src)} done in {time.time() - t:.0f} s"
                         + (("\n" + out) if out.strip() else ""))
                return obj

            with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
                objs = list(ex.map(one, srcs))
            tmp = os.path.join(work, name)
            _run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp, *objs])
            final = os.path.join(d, name)
            os.replace(tmp, final)
            for old in glob.glob(os.path.join(d, "gl3hip-*.so")):
                if old != final:
                    try:
                        os.remove(old)
                    except OSError:
                        pass
            if verbose:
                _say(f"built {final} in {time.time() - t0:.0f} s")
            return final
        finally:
            shutil.rmtree(work, ignore_errors=True)
    raise RuntimeError(f"no writable folder for the HIP library ({last_error})")


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
