"""Builds libcatccos_mx.so (HIP kernels + C ABI) for gfx950 with hipcc.

Usage: python -m catccos_amd.build [--verbose] [--jobs N]
Objects go to catccos_amd/_build/, the library to catccos_amd/lib/.  Sources are
rebuilt when they or any header are newer than the object (``force`` rebuilds all).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libcatccos_mx.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime() -> float:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(ROOT, "include", "catccos_mx.h"))
    return max(os.path.getmtime(h) for h in hs)


def _filter(text: str) -> str:
    keep = [ln for ln in text.splitlines()
            if "packed-fp32-ops' is not a recognized feature" not in ln and ln.strip()]
    return "\n".join(keep)


def compile_object(path: str, obj: str, extra_flags=(), verbose: bool = False) -> str:
    """hipcc -c of one .hip file with the library's flags (plus ``extra_flags``)."""
    cmd = [HIPCC, *FLAGS, *extra_flags, "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = _filter(r.stdout + r.stderr)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {path}:\n{out}")
    if verbose and out:
        print(out)
    return obj


def link_shared(lib: str, objs) -> str:
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + _filter(r.stdout + r.stderr))
    return lib


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = _filter(r.stdout + r.stderr)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    if verbose and out:
        print(out)
    return obj


def build(force: bool = False, verbose: bool = False, jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    hm = _headers_mtime()
    todo, objs = [], []
    for s in sources():
        obj = os.path.join(OBJ, s[:-4] + ".o")
        objs.append(obj)
        stale = (force or not os.path.exists(obj)
                 or os.path.getmtime(obj) < max(os.path.getmtime(os.path.join(CSRC, s)), hm))
        if stale:
            todo.append(s)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(lambda s: _compile(s, verbose), todo))
    if todo or not os.path.exists(LIB):
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs],
                           capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + _filter(r.stdout + r.stderr))
    return LIB


if __name__ == "__main__":
    force = "--force" in sys.argv
    verbose = "--verbose" in sys.argv
    print(build(force=force, verbose=verbose))
