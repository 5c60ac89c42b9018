"""Compiles the HIP sources of this folder for gfx950 into one shared library per activation type.

The library lies in ``csrc/_build/`` next to the sources (or, where that folder cannot be written,
in a per-user folder under the temporary directory) and carries a hash of its sources and flags in
its name, so a library built from other sources is never loaded by mistake.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

CSRC = os.path.dirname(os.path.abspath(__file__))

# sources per activation type: each has matrix-core kernels of its own
# (host/: the step executor and its way into the vendor's matrix library, host code that calls the kernels' entry points)
COMMON_SOURCES = ["elementwise.hip", "gemm_generic.hip", "attention_generic.hip", "moe.hip", "sampling.hip",
                  "host/engine.cpp", "host/vendor.cpp"]
SOURCES = {
    "float32": COMMON_SOURCES + ["gemm_f32.hip", "attention_f32.hip"],
    "bfloat16": COMMON_SOURCES + ["gemm_mfma.hip", "attention_mfma.hip", "probe.hip"],
}
HEADERS = ["common.h", "gates.def", "no_alloc.h", "gemm_mfma.h", "turboquant_kernels.h", "host/engine.h", "host/vendor.h",
           "host/host_common.h"]
DEFINES = {"float32": "-DTQ_ACT_F32", "bfloat16": "-DTQ_ACT_BF16"}
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-fno-gpu-rdc",
         # keep the compiler from forming packed 32-bit float instructions
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


class BuildError(RuntimeError):
    pass


def _existing(names):
    return [n for n in names if os.path.isfile(os.path.join(CSRC, n))]


def _hash(dtype: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + [DEFINES[dtype]]).encode())
    for name in _existing(SOURCES[dtype]) + _existing(HEADERS):
        h.update(name.encode())
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def _build_dirs() -> list[str]:
    return [os.path.join(CSRC, "_build"),
            os.path.join(tempfile.gettempdir(), f"turboquant_cpp_amd_build_{os.getuid()}")]


def library_name(dtype: str) -> str:
    return f"libtq_{dtype}-{_hash(dtype)}.so"


def find_library(dtype: str) -> str | None:
    """The built library that matches the present sources, or None."""
    name = library_name(dtype)
    for d in _build_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc): the gfx950 kernels cannot be built")


def _writable_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the built library: tried " + ", ".join(_build_dirs()))


def build(dtype: str, force: bool = False, verbose: bool = True) -> str:
    """Compiles the library for one activation type and returns its path."""
    if dtype not in SOURCES:
        raise BuildError(f"unknown activation type {dtype!r}")
    if not force:
        found = find_library(dtype)
        if found:
            return found
    hipcc = _hipcc()
    out_dir = _writable_dir()
    target = os.path.join(out_dir, library_name(dtype))
    obj_dir = os.path.join(out_dir, f"obj_{dtype}_{os.getpid()}")
    os.makedirs(obj_dir, exist_ok=True)
    say = (lambda m: print(f"[turboquant] {m}", file=sys.stderr, flush=True)) if verbose else (lambda m: None)
    sources = _existing(SOURCES[dtype])
    say(f"compiling {len(sources)} HIP sources for gfx950 ({dtype}) into {target}")
    t0 = time.time()
    procs = []
    for src in sources:
        obj = os.path.join(obj_dir, os.path.splitext(os.path.basename(src))[0] + ".o")
        cmd = [hipcc, *FLAGS, DEFINES[dtype], "-c", os.path.join(CSRC, src), "-o", obj]
        # what the compiler prints goes to a file: a pipe that nobody reads while the compilers run together
        # would block the one that fills it
        log = open(obj + ".log", "w+")
        procs.append((src, obj, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT), log))
    objs = []
    pending = list(procs)
    last = time.time()
    while pending:
        for item in list(pending):
            src, obj, p, log = item
            if p.poll() is None:
                continue
            log.seek(0)
            out = log.read()
            log.close()
            pending.remove(item)
            if p.returncode != 0:
                for _, _, q, _ in pending:
                    q.kill()
                raise BuildError(f"hipcc failed on {src}:\n{out}")
            say(f"  compiled {src} ({time.time() - t0:.0f}s)")
            objs.append(obj)
        if pending:
            time.sleep(0.2)
            if time.time() - last > 10:
                say(f"  still compiling: {', '.join(s for s, _, _, _ in pending)} ({time.time() - t0:.0f}s)")
                last = time.time()
    tmp = target + f".tmp{os.getpid()}"
    link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *sorted(objs), "-ldl", "-o", tmp],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if link.returncode != 0:
        raise BuildError(f"hipcc failed to link {target}:\n{link.stdout}")
    os.replace(tmp, target)
    shutil.rmtree(obj_dir, ignore_errors=True)
    for old in os.listdir(out_dir):     # what a build that was killed left behind
        pid = old.rsplit("_", 1)[-1]
        if old.startswith("obj_") and pid.isdigit() and not os.path.exists(f"/proc/{pid}"):
            shutil.rmtree(os.path.join(out_dir, old), ignore_errors=True)
    for old in os.listdir(out_dir):     # libraries of earlier sources
        if old.startswith(f"libtq_{dtype}-") and old.endswith(".so") and old != os.path.basename(target):
            try:
                os.remove(os.path.join(out_dir, old))
            except OSError:
                pass
    say(f"built {os.path.basename(target)} in {time.time() - t0:.0f}s")
    return target


RUNNER_SOURCES = ["host/quant_main.cpp", "host/engine.h", "gates.def"]


def runner_name() -> str:
    h = hashlib.sha256()
    for name in RUNNER_SOURCES:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    return f"tq_run-{h.hexdigest()[:12]}"


def find_runner() -> str | None:
    for d in _build_dirs():
        p = os.path.join(d, runner_name())
        if os.path.isfile(p):
            return p
    return None


def build_runner(force: bool = False, verbose: bool = True) -> str:
    """Compiles the host program without Python (host/quant_main.cpp) and returns its path.  It loads a kernel
    library at run time and is linked against the HIP runtime only."""
    if not force:
        found = find_runner()
        if found:
            return found
    hipcc = _hipcc()
    target = os.path.join(_writable_dir(), runner_name())
    tmp = target + f".tmp{os.getpid()}"
    if verbose:
        print(f"[turboquant] compiling the host program into {target}", file=sys.stderr, flush=True)
    run = subprocess.run([hipcc, "-O2", "-std=c++17", os.path.join(CSRC, "host", "quant_main.cpp"), "-ldl", "-o", tmp],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if run.returncode != 0:
        raise BuildError(f"hipcc failed on host/quant_main.cpp:\n{run.stdout}")
    os.replace(tmp, target)
    for old in os.listdir(os.path.dirname(target)):
        if old.startswith("tq_run-") and old != os.path.basename(target) and ".tmp" not in old:
            try:
                os.remove(os.path.join(os.path.dirname(target), old))
            except OSError:
                pass
    return target


def build_all(force: bool = True, verbose: bool = True) -> list[str]:
    return [build(d, force=force, verbose=verbose) for d in SOURCES] + [build_runner(force=force, verbose=verbose)]


if __name__ == "__main__":
    for path in build_all():
        print(path)
