"""Seeded synthetic inputs for the benchmark configurations (numpy only).

Every generator takes an explicit seed and draws from
``numpy.random.Generator(PCG64(seed))`` so a CPU checker and the GPU path see the
same tensors.  bf16 tensors are returned as uint16 bit patterns.
"""
from __future__ import annotations

import numpy as np


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16).reshape(x.shape)


def activations_with_outliers(m: int, k: int, seed: int, outlier_frac: float = 1e-3, outlier_scale: float = 100.0):
    """bf16 [m, k]: N(0,1) with a Bernoulli(outlier_frac) mask of elements scaled
    by outlier_scale (block-quantization stress: one outlier sets a block's scale)."""
    r = _rng(seed)
    x = r.standard_normal((m, k), dtype=np.float32)
    mask = r.random((m, k), dtype=np.float32) < outlier_frac
    x[mask] *= np.float32(outlier_scale)
    return f32_to_bf16_bits(x)


def normal_bf16(shape, seed: int, std: float = 1.0):
    return f32_to_bf16_bits(_rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(std))


def zipf_routing(tokens: int, experts: int, top_k: int, seed: int, s: float = 1.1, empty: int = 2):
    """int32 [tokens, top_k]: per token top_k distinct experts drawn without
    replacement with p_e proportional to 1/rank(e)^s over a seeded permutation of
    the experts; the ``empty`` lowest-ranked experts get p = 0 (ragged group sizes
    with empty groups, deterministically)."""
    r = _rng(seed)
    perm = r.permutation(experts)
    p = 1.0 / np.arange(1, experts + 1, dtype=np.float64) ** s
    if empty:
        p[experts - empty:] = 0.0
    p /= p.sum()
    prob = np.zeros(experts)
    prob[perm] = p
    # Gumbel top-k == sampling without replacement proportional to prob
    g = r.gumbel(size=(tokens, experts))
    with np.errstate(divide="ignore"):
        keys = np.log(prob)[None, :] + g
    idx = np.argsort(-keys, axis=1, kind="stable")[:, :top_k]
    return idx.astype(np.int32)


def softmax_topk_routing(tokens: int, experts: int, top_k: int, seed: int):
    """(expert_idx int32 [tokens, top_k], weights fp32 [tokens, top_k]): top-k of a
    softmax over N(0,1) logits, weights renormalised to sum to 1 (fp32)."""
    r = _rng(seed)
    logits = r.standard_normal((tokens, experts), dtype=np.float32)
    z = np.exp(logits - logits.max(axis=1, keepdims=True), dtype=np.float32)
    p = (z / z.sum(axis=1, keepdims=True)).astype(np.float32)
    idx = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    w = np.take_along_axis(p, idx, axis=1)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return idx.astype(np.int32), w


def random_codes_e4m3(shape, seed: int, exp_lo: int = 0x20, exp_hi: int = 0x58):
    """Uniform random E4M3 codes with biased magnitude field in [exp_lo, exp_hi)
    and random sign - cheap stand-in for quantized weights when only throughput
    matters (never NaN)."""
    r = _rng(seed)
    mag = r.integers(exp_lo, exp_hi, size=shape, dtype=np.uint8)
    sign = (r.integers(0, 2, size=shape, dtype=np.uint8) << 7).astype(np.uint8)
    return mag | sign
