"""Builds the HIP library of return_amd with hipcc for gfx950 and finds it again.

Sources are return_amd/csrc/*.hip. The library is kept in-tree (return_amd/_lib/); if that
folder cannot be written, in a per-user folder under the temporary directory. A stored
hash of sources and flags decides whether what is there is still current, so a fresh
checkout compiles at its first call and prints a line now and then while it does.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
LIB_NAME = "libreturn_amd.so"

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[return_amd] {msg}", file=sys.stderr, flush=True)


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def compile_units():
    """(source, defines, object name): a source with a line '// BUILD-VARIANTS: A=1 B=2 ...' is
    compiled once per listed define (large template families are split to compile in parallel)."""
    units = []
    for src in sources():
        base = os.path.basename(src)[:-4]
        variants = []
        with open(src) as f:
            for line in f:
                if line.startswith("// BUILD-VARIANTS:"):
                    variants = line.split(":", 1)[1].split()
                    break
        if not variants:
            units.append((src, [], base + ".o"))
        for v in variants:
            units.append((src, ["-D" + v], f"{base}.{v.replace('=', '_')}.o"))
    return units


def _headers():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    for path in sources() + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _lib_dirs():
    yield os.path.join(os.path.dirname(_HERE), "_lib")
    yield os.path.join(tempfile.gettempdir(), f"return_amd-{os.getuid()}", "_lib")


def _writable_dir():
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the HIP library: tried " + ", ".join(_lib_dirs()))


def find_current():
    """Path of a built library that matches the sources, or None."""
    want = source_hash()
    for d in _lib_dirs():
        lib, stamp = os.path.join(d, LIB_NAME), os.path.join(d, LIB_NAME + ".hash")
        if os.path.exists(lib) and os.path.exists(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return lib
    return None


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise BuildError("hipcc not found: the HIP kernels of return_amd cannot be built")
    return exe


def _run(cmd, what):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise BuildError(f"{what} failed:\n{' '.join(cmd)}\n{p.stdout}")
    return p.stdout


def build(force: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    if not force:
        have = find_current()
        if have:
            return have
    hipcc = _hipcc()
    out_dir = _writable_dir()
    # objects in a folder of this process's own: two processes that build at once (two first
    # calls in a fresh checkout) do not write, link or delete each other's files
    obj_dir = tempfile.mkdtemp(prefix="_build-", dir=out_dir)
    units = compile_units()
    t0 = time.time()
    _say(f"compiling {len(units)} HIP units for {ARCH} into {out_dir}")
    done = threading.Event()

    def heartbeat():
        while not done.wait(15.0):
            _say(f"still compiling ({time.time() - t0:.0f} s)")

    threading.Thread(target=heartbeat, daemon=True).start()
    try:
        def one(unit):
            src, defines, name = unit
            obj = os.path.join(obj_dir, name)
            _run([hipcc, *FLAGS, *defines, "-c", src, "-o", obj], f"compiling {name}")
            _say(f"compiled {name[:-2]} ({time.time() - t0:.0f} s)")
            return obj
        workers = min(len(units), max(1, min(8, os.cpu_count() or 1)))
        with concurrent.futures.ThreadPoolExecutor(workers) as pool:
            objs = list(pool.map(one, units))
        tmp = os.path.join(out_dir, f".{LIB_NAME}.{os.path.basename(obj_dir)}")
        _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs], "linking")
        lib = os.path.join(out_dir, LIB_NAME)
        os.replace(tmp, lib)
        with open(tmp + ".hash", "w") as f:
            f.write(source_hash())
        os.replace(tmp + ".hash", lib + ".hash")
    finally:
        done.set()
        shutil.rmtree(obj_dir, ignore_errors=True)
    _say(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def ensure_built() -> str:
    """The current library, compiled now if there is none."""
    return build(force=False)
