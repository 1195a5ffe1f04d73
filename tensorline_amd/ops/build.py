"""Builds the HIP kernels into one shared library for gfx950, and finds it again.

``hipcc`` compiles each ``csrc/*.hip`` file to an object and links them into
``libtensorline_hip.so`` next to this file (or, when that folder cannot be written, under the
temporary folder).  A stamp file records the hash of the sources a library was built from; a
library whose stamp does not match the sources is rebuilt on load, so stale code is never run.
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

OFFLOAD_ARCH = "gfx950"
LIB_NAME = "libtensorline_hip.so"

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")

# -packed-fp32-ops off: the compiler otherwise forms packed float instructions from scalar code.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-unused-result",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for path in sources() + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _candidate_dirs() -> list[str]:
    out = [_HERE]
    tmp = os.environ.get("TMPDIR") or tempfile.gettempdir()
    out.append(os.path.join(tmp, f"tensorline_amd-{os.getuid()}"))
    return out


def _stamp_ok(lib: str, want: str) -> bool:
    try:
        with open(lib + ".stamp", "r", encoding="utf-8") as f:
            return f.read().strip() == want
    except OSError:
        return False


def find_built() -> str | None:
    """Path of a library that matches the current sources, or None."""
    want = source_hash()
    for d in _candidate_dirs():
        lib = os.path.join(d, LIB_NAME)
        if os.path.isfile(lib) and _stamp_ok(lib, want):
            return lib
    return None


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


def _writable_dir() -> str:
    for d in _candidate_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.unlink(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the built kernels (tried: %s)" % ", ".join(_candidate_dirs()))


def _say(msg: str, verbose: bool) -> None:
    if verbose:
        print(f"[tensorline_amd build] {msg}", file=sys.stderr, flush=True)


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Compile every source for gfx950 and link the library.  Always compiles.  Returns its path."""
    hipcc = find_hipcc()
    out_dir = _writable_dir()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise BuildError(f"no .hip sources under {CSRC}")
    want = source_hash()
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)      # hipcc wants a home folder for its caches; any writable one does
    t0 = time.time()
    _say(f"compiling {len(srcs)} HIP sources for {OFFLOAD_ARCH} with {hipcc} (about a minute)", verbose)

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
        proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
        last = time.time()
        while True:
            try:
                out, _ = proc.communicate(timeout=15)
                break
            except subprocess.TimeoutExpired:
                if time.time() - last >= 15:
                    _say(f"still compiling {os.path.basename(src)} ({time.time() - t0:.0f} s)", verbose)
                    last = time.time()
        if proc.returncode != 0:
            raise BuildError(f"hipcc failed on {src}:\n{out}")
        _say(f"compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)", verbose)
        return obj

    workers = jobs or min(len(srcs), max(1, min(8, (os.cpu_count() or 2))))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objs = list(pool.map(compile_one, srcs))

    lib = os.path.join(out_dir, LIB_NAME)
    tmp_lib = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", *objs, "-o", tmp_lib]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    if res.returncode != 0:
        raise BuildError(f"linking {LIB_NAME} failed:\n{res.stdout}")
    os.replace(tmp_lib, lib)
    with open(lib + ".stamp", "w", encoding="utf-8") as f:
        f.write(want + "\n")
    _say(f"built {lib} in {time.time() - t0:.0f} s", verbose)
    return lib


def ensure_built(verbose: bool = True) -> str:
    """The library for the current sources: the built one if there is one, else build it now."""
    lib = find_built()
    if lib is not None:
        return lib
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
