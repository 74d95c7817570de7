#!/usr/bin/env python3
"""Checks the compiled form of the hand-scheduled matmul kernels (mx_gemm_pipe.h, mx_gemm_pipe_fp4.h, mx_gemm_wreg.h).

The instruction stream between a kernel's first and last MFMA is written out by hand, one instruction per asm
statement; the compiler adds the address arithmetic around it and allocates the registers.  Two things it may also
add are fatal for the schedule and invisible in the source:

* a spill or reload (``scratch_*``) inside that stream, and
* a wait for vector memory (``s_waitcnt vmcnt(N)``) that is not one of the schedule's own: the compiler puts one
  behind every reload of a spilled value, also when the reload sits before the loop and the first use inside it,
  and such a wait drains the operand loads that the schedule keeps in flight.

A third check concerns correctness: an LDS-DMA load (``buffer_load ... lds``) takes its LDS address from M0, and the
kernels that issue it in two statements (write of M0, a scheduled instruction in the wait state, the load) rely on
nothing else writing M0 in between and on at least one instruction standing there.

For every instantiation that the library dispatches to, this script compiles that one kernel to assembly
(device only, nothing is linked or run) and reports the spills and waits found between the first and the last
MFMA.  Run it after any change to the kernels, the epilogues or their helpers:

    python3 tests/check_pipe_schedule.py          # a few seconds per kernel

Exit status 0 when every kernel is clean.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HERE = os.path.join(ROOT, "catccos_amd", "csrc")          # where the kernel sources live
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         f"-I{os.path.join(ROOT, 'include')}", f"-I{HERE}", "-S", "--cuda-device-only", "-Wno-unused-command-line-argument"]

# (explicit instantiation, the schedule's own vmcnt waits inside the stream: the early tile loads -- 7 or 8 (6 for FP4); the
# persistent 2 x 2 kernels send all 8 weight loads early -- plus 2 prefetch loads in the persistent 2 x 2 kernels)
#   mx_gemm_pipe_kernel<FMT, EPI, TM, WW, WM, NSLOT>; EPI 0 store, 1 SwiGLU + requant, 2 lean bf16, 4 lean fp16, 5 = 1 + bf16 activations
#   mx_gemm_pipe_fp4_kernel<EPI, WW, WM>
#   mx_gemm_wreg_kernel<FMT, EPI, TM>: the wait at the start of a slab leaves the weight loads of the next slab and all loads of
#   the one after in flight (8 + 16 or 17), and behind the slab that sent a scale block the loads of that block too
KERNELS = [
    ("mx_gemm_wreg_kernel<0, 1, 256>", {24, 26}),
    ("mx_gemm_wreg_kernel<0, 2, 256>", {24, 26}),
    ("mx_gemm_wreg_kernel<0, 4, 256>", {24, 26}),
    ("mx_gemm_wreg_kernel<1, 2, 256>", {24, 26}),
    ("mx_gemm_wreg_kernel<1, 4, 256>", {24, 26}),
    ("mx_gemm_wreg_kernel<0, 1, 288>", {25, 29}),               # nine activation loads per slab; four loads go out with a scale block
    ("mx_gemm_wreg_kernel<0, 2, 288>", {25, 29}),
    ("mx_gemm_wreg_kernel<0, 4, 288>", {25, 29}),
    ("mx_gemm_wreg_kernel<1, 2, 288>", {25, 29}),
    ("mx_gemm_wreg_kernel<1, 4, 288>", {25, 29}),
    ("mx_gemm_pipe_kernel<0, 1, 256, 2, 2, 2>", {10}),
    ("mx_gemm_pipe_kernel<0, 1, 256, 4, 1, 2>", {8}),
    ("mx_gemm_pipe_kernel<0, 5, 256, 2, 2, 2>", {10}),          # SwiGLU + requant that also writes the bf16 activations
    ("mx_gemm_pipe_kernel<0, 5, 256, 4, 1, 2>", {8}),
    ("mx_gemm_pipe_kernel<0, 2, 256, 2, 2, 2>", {10}),
    ("mx_gemm_pipe_kernel<0, 4, 256, 2, 2, 2>", {10}),
    ("mx_gemm_pipe_kernel<0, 0, 256, 2, 2, 2>", {7}),
    ("mx_gemm_pipe_kernel<0, 0, 256, 4, 1, 2>", {8}),
    ("mx_gemm_pipe_kernel<0, 0, 128, 4, 1, 3>", {14}),
    ("mx_gemm_pipe_kernel<0, 1, 128, 4, 1, 3>", {14}),
    ("mx_gemm_pipe_fp4_kernel<2, 2, 2>", {10}),
    ("mx_gemm_pipe_fp4_kernel<4, 2, 2>", {10}),
    ("mx_gemm_pipe_fp4_kernel<2, 4, 1>", {8}),
    ("mx_gemm_pipe_fp4_kernel<4, 4, 1>", {8}),
    ("mx_gemm_pipe_fp4_kernel<0, 2, 2>", {6}),
    ("mx_gemm_pipe_fp4_kernel<0, 4, 1>", {8}),
]


def prefix_source() -> str:
    """mx_gemm.hip up to and including the kernel headers (everything a kernel needs, no host code)."""
    text = open(os.path.join(HERE, "mx_gemm.hip")).read()
    marker = '#include "mx_gemm_pipe_fp4.h"\n'
    return text[: text.index(marker) + len(marker)]


def check(kernel: str, own_waits: set[int], workdir: str) -> list[str]:
    src = os.path.join(workdir, "one_kernel.hip")
    asm = os.path.join(workdir, "one_kernel.s")
    with open(src, "w") as f:
        f.write(prefix_source())
        f.write(f"template __global__ void {kernel}(const GemmParams);\n}}\n}}\n")
    r = subprocess.run([HIPCC, *FLAGS, "-o", asm, src], capture_output=True, text=True)
    if r.returncode != 0:
        return ["does not compile:\n" + r.stderr[-2000:]]
    lines = [ln.strip() for ln in open(asm)]
    mfma = [i for i, ln in enumerate(lines) if ln.startswith("v_mfma")]
    if not mfma:
        return ["no MFMA found"]
    problems = []
    code = [ln for ln in lines if ln and not ln.startswith(";")]
    for i, ln in enumerate(code):
        if ln.startswith("buffer_load") and ln.endswith(" lds"):
            j = i - 1
            while j >= 0 and not re.search(r"\bm0\b", code[j]):
                j -= 1
            between = [x for x in code[j + 1: i] if not x.endswith(":")]
            labels = [x for x in code[j + 1: i] if x.endswith(":") and not x.startswith(".Lskip")]      # the MFMA-skip branches are local
            if j < 0 or not code[j].startswith("s_mov_b32 m0") or not between or labels:
                problems.append("LDS-DMA load without its own M0 write and wait state: " + ln)
    for ln in lines[mfma[0]: mfma[-1] + 1]:
        if ln.startswith("scratch_"):
            problems.append("spill traffic inside the scheduled stream: " + ln)
        m = re.match(r"s_waitcnt\b.*vmcnt\((\d+)\)", ln)
        if m and int(m.group(1)) not in own_waits:
            problems.append("a wait that is not the schedule's own: " + ln)
    return problems


def main() -> int:
    bad = 0
    with tempfile.TemporaryDirectory() as workdir:
        for kernel, own in KERNELS:
            problems = check(kernel, own, workdir)
            print(("ok      " if not problems else "FAILED  ") + kernel, flush=True)
            for p in problems[:8]:
                print("        " + p)
            bad += bool(problems)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
