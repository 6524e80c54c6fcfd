"""Compiles the HIP sources of this folder for gfx950 into one shared library.

``hipcc`` is called directly (no extension machinery): each ``.hip`` file
becomes an object, the objects are linked into ``libkllm_hip.so``.  The library
is kept in ``_build/`` next to the sources, together with a stamp of the
sources it was built from; ``ensure_built()`` rebuilds when the stamp differs
and otherwise only returns the path.  Where the source tree cannot be written,
a per-user folder under the system's temporary folder is used instead.
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

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libkllm_hip.so"
ARCH = "gfx950"
# Packed 32-bit float instructions are switched off for all device code.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result"]


class BuildError(RuntimeError):
    pass


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def _stamp() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(HERE)):
        if name.endswith((".hip", ".hpp", ".h")):
            h.update(name.encode())
            with open(os.path.join(HERE, name), "rb") as f:
                h.update(f.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _writable_build_dir() -> str:
    d = os.path.join(HERE, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"kllm_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _candidates():
    yield os.path.join(HERE, "_build")
    yield os.path.join(tempfile.gettempdir(), f"kllm_amd_build_{os.getuid()}")


def built_library():
    """Path of an up-to-date library, or None."""
    want = _stamp()
    for d in _candidates():
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, "stamp")
        if os.path.exists(lib) and os.path.exists(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def _log(msg):
    print(f"[kllm_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose=True) -> str:
    """Compile everything, whether or not a library exists.  Returns its path."""
    hipcc = _hipcc()
    out_dir = _writable_build_dir()
    env = dict(os.environ)
    # hipcc keeps temporary files; give it a place when HOME is empty or unset.
    env.setdefault("TMPDIR", tempfile.gettempdir())
    srcs = sources()
    t0 = time.time()
    if verbose:
        _log(f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(src):
        obj = os.path.join(out_dir, src[:-4] + ".o")
        cmd = [hipcc, *FLAGS, "-I", HERE, "-c", os.path.join(HERE, src), "-o", obj]
        t = time.time()
        p = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        if p.returncode != 0:
            raise BuildError(f"hipcc failed on {src}:\n{p.stderr[-4000:]}")
        if verbose:
            _log(f"  {src} done in {time.time() - t:.1f} s")
        return obj

    workers = max(1, min(len(srcs), (os.cpu_count() or 2), 8))
    with ThreadPoolExecutor(workers) as ex:
        objs = list(ex.map(compile_one, srcs))
    lib_tmp = os.path.join(out_dir, LIB_NAME + f".{os.getpid()}.tmp")
    cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", lib_tmp]
    p = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if p.returncode != 0:
        raise BuildError(f"linking failed:\n{p.stderr[-4000:]}")
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(lib_tmp, lib)
    with open(os.path.join(out_dir, "stamp"), "w") as f:
        f.write(_stamp())
    if verbose:
        _log(f"built {lib} in {time.time() - t0:.1f} s")
    return lib


def ensure_built(verbose=True) -> str:
    """The library's path; compiles first if no up-to-date library exists."""
    return built_library() or build(verbose)


if __name__ == "__main__":
    print(build())
