#!/usr/bin/env python3
"""Builds tests/lib/libcatccos_mx_test.so: the library with the test hooks that the product does not carry.

It is the product library's own objects, except that mx_gemm.hip is compiled once more with -DCMX_TEST_HOOKS
(cmx_debug_force_tile / cmx_debug_disable_streaming: pin the tile shape or force the register-staged kernels so
that tests reach every compiled instantiation), plus tests/csrc/*.hip (cmx_mfma_raw_probe: one MFMA on
caller-supplied registers, for the register-layout known-answer tests).

    python tests/build_test_lib.py        # after `python -m catccos_amd.build`
"""
from __future__ import annotations

import os
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from catccos_amd import build as B  # noqa: E402

TEST_CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "lib", "libcatccos_mx_test.so")


def build(force: bool = False) -> str:
    B.build()                                              # the product objects this library shares
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    jobs = [(os.path.join(B.CSRC, "mx_gemm.hip"), os.path.join(OBJ, "mx_gemm_hooks.o"), ("-DCMX_TEST_HOOKS",))]
    for f in sorted(os.listdir(TEST_CSRC)):
        if f.endswith(".hip"):
            jobs.append((os.path.join(TEST_CSRC, f), os.path.join(OBJ, f[:-4] + ".o"), ()))
    newest_header = B._headers_mtime()
    todo = [j for j in jobs if force or not os.path.exists(j[1])
            or os.path.getmtime(j[1]) < max(os.path.getmtime(j[0]), newest_header)]
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(lambda j: B.compile_object(j[0], j[1], j[2]), todo))
    shared = [os.path.join(B.OBJ, s[:-4] + ".o") for s in B.sources() if s != "mx_gemm.hip"]
    objs = [j[1] for j in jobs] + shared
    if todo or not os.path.exists(LIB) or os.path.getmtime(LIB) < max(os.path.getmtime(o) for o in objs):
        B.link_shared(LIB, objs)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
