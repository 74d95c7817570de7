"""CPU oracle for the INT8 W8A8 dispatch + grouped matmul + dequant + SwiGLU path (TEST INFRASTRUCTURE - never
on the product path; only tests, the smoke check and the benchmark's CPU leg may import it).

Restates, in plain numpy, what examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py computes for the
reference operator DispatchGmmDequantSwiglu: per-token dynamic INT8 quantisation of the routed activations,
INT8 x INT8 -> INT32 grouped matmul over experts, per-channel dequant to fp16, per-token dequant in fp32, SwiGLU.
Every function cites the lines it follows.

Pinning status (tests/test_oracle_int8.py): the INT32 matmul is exact integer arithmetic (checked against Python
integers), the fp16 rounding is numpy's IEEE conversion (checked against torch's), the whole chain is checked
against an independent torch CPU formulation built from library ops (``matmul`` on int32, ``.half()``,
``torch.sigmoid``).  The per-token quantiser follows the generator's ``quant`` helper (:269-274); the generator
itself obtains its INT8 activations from an NPU-only library routine (``torch_npu.npu_moe_init_routing_v2`` with
``quant_mode=1``, :159-165) whose source is not in the tree, so bit-equality of the INT8 codes with that routine is
"parity unpinned" -- everything downstream takes the codes and scales as given and is pinned.
"""
from __future__ import annotations

import numpy as np


def dynamic_quant(x) -> tuple[np.ndarray, np.ndarray]:
    """Per-row symmetric INT8 quantisation: ``q = round(x * 127 / rowmax)``, ``scale = rowmax / 127`` in fp32,
    round half to even (``torch.round``).  gen_data_dispatch_gmm_dequant_swiglu.py:269-274.
    A row of zeros (where the generator's formula divides 0 by 0) gives codes 0 and scale 0."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rowmax = np.abs(x).max(axis=-1)
    safe = np.where(rowmax > 0, rowmax, np.float32(1)).astype(np.float32)
    scaled = (x * np.float32(127.0)).astype(np.float32) / safe[..., None]
    q = np.rint(scaled.astype(np.float32)).astype(np.int32)
    q = np.where(rowmax[..., None] > 0, q, 0).astype(np.int8)
    scale = (rowmax / np.float32(127.0)).astype(np.float32)
    return q, scale


def dispatch_quant(x, sorted2src, top_k: int) -> tuple[np.ndarray, np.ndarray]:
    """Routed activations: row i of the result is token ``sorted2src[i] // top_k`` quantised by
    :func:`dynamic_quant` (the expanded, expert-sorted INT8 matrix and its per-token scales that the generator
    takes from the routing routine, :159-176)."""
    q, s = dynamic_quant(x)
    tok = np.asarray(sorted2src, dtype=np.int64) // top_k
    return q[tok], s[tok]


def swiglu(x) -> np.ndarray:
    """``x0 * sigmoid(x0) * gate`` with x0 = first half of the columns, gate = second half, fp32.  :263-267"""
    x = np.asarray(x, dtype=np.float32)
    half = x.shape[-1] // 2
    x0, gate = x[..., :half], x[..., half:]
    sig = (np.float32(1) / (np.float32(1) + np.exp(-x0.astype(np.float32)))).astype(np.float32)
    return ((x0 * sig).astype(np.float32) * gate).astype(np.float32)


def gmm_dequant_swiglu(a, tok_scale, b, ch_scale, counts) -> np.ndarray:
    """a int8 [rows, K] (expert-sorted), tok_scale fp32 [rows], b int8 [E, K, N], ch_scale fp32 [E * N] (expert
    major), counts rows per expert -> fp32 [rows, N / 2].

    Per expert (:291-320): ``c = a_g.int32 @ b_g.int32``; ``h = fp16(fp32(c) * ch_scale_g)``;
    ``y = fp32(h) * tok_scale[:, None]``; ``out = swiglu(y)``.  The offset the generator adds is all zeros (:83-85).
    """
    a = np.asarray(a, dtype=np.int8)
    b = np.asarray(b, dtype=np.int8)
    e, k, n = b.shape
    ch = np.asarray(ch_scale, dtype=np.float32).reshape(e, n)
    ts = np.asarray(tok_scale, dtype=np.float32)
    rows = a.shape[0]
    out = np.zeros((rows, n // 2), dtype=np.float32)
    r0 = 0
    for g, cnt in enumerate(np.asarray(counts, dtype=np.int64)):
        if cnt == 0:
            continue
        c = a[r0:r0 + cnt].astype(np.int32) @ b[g].astype(np.int32)          # exact: |sum| < 2^31 for K < 2^17
        h = (c.astype(np.float32) * ch[g][None, :]).astype(np.float32).astype(np.float16)
        y = (h.astype(np.float32) * ts[r0:r0 + cnt, None]).astype(np.float32)
        out[r0:r0 + cnt] = swiglu(y)
        r0 += cnt
    return out


def channel_scale_words(ch_scale) -> np.ndarray:
    """The generator's scale file: one int64 per channel whose low 32 bits are the fp32 scale (:70-73)."""
    ch = np.ascontiguousarray(ch_scale, dtype=np.float32).reshape(-1)
    words = np.zeros(ch.size, dtype=np.int64)
    words.view(np.float32)[0::2] = ch
    return words


def truncate_scale(x) -> np.ndarray:
    """The generator keeps 19 bits of its random per-channel scales: ``(bits >> 13) << 13`` (:71)."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.int32)
    return ((bits >> 13) << 13).view(np.float32)
