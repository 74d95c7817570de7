"""Cross-checks the two CPU restatements (numpy and C) against each other, and the oracle's
sizing formulas against the reference's own header where oracle/_ref has been built."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from oracle import mx_oracle as O
from catccos_amd import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(HERE), "oracle")
LIBC = os.path.join(ORACLE_DIR, "libmx_oracle.so")
LIBREF = os.path.join(ORACLE_DIR, "_ref", "libmoe_ub_ref.so")
REFBIN = os.path.join(ORACLE_DIR, "_ref", "test_moe_ub_capacity")


@pytest.fixture(scope="module")
def libc():
    if not os.path.exists(LIBC):
        subprocess.run(["make", "-C", ORACLE_DIR, LIBC], check=True, capture_output=True)
    return C.CDLL(LIBC)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("fmt,fi", [("E4M3", 0), ("E5M2", 1), ("E2M1", 2)])
@pytest.mark.parametrize("mode,mi", [("rne", 0), ("lut", 1)])
def test_c_quantizer_equals_numpy(libc, fmt, fi, mode, mi):
    xb = W.activations_with_outliers(48, 200, seed=fi * 2 + mi)          # ragged: 200 = 6 blocks + 8
    tab = {"E4M3": O.e4m3_table()[:127], "E5M2": O.e5m2_table()[:124], "E2M1": O.fp4_table()[:8]}[fmt]
    mid = ((tab[:-1].astype(np.float64) + tab[1:]) / 2).astype(np.float32)
    mid = mid[O.bf16_round(mid) == mid][:150]
    x2 = np.zeros((mid.size, 200), dtype=np.float32)
    x2[:, 0] = 2.0 ** O.FORMATS[fmt]["emax"]
    x2[:, 1] = mid
    x2[:, 2] = -mid
    xb = np.concatenate([xb, O.f32_to_bf16_bits(x2)])
    rows, cols = xb.shape
    codes = np.zeros((rows, cols), dtype=np.uint8)
    scales = np.zeros((rows, O.scale_cols(cols)), dtype=np.uint8)
    assert libc.mxo_quant_bf16(_p(np.ascontiguousarray(xb)), rows, cols, fi, mi, _p(codes), _p(scales)) == 0
    q, s = O.mx_quant_bf16(xb, fmt, mode)
    assert np.array_equal(scales, s)
    assert np.array_equal(codes, q)
    out = np.zeros((rows, cols), dtype=np.float32)
    libc.mxo_dequant(_p(codes), _p(scales), rows, cols, fi, _p(out))
    assert np.array_equal(out, O.mx_dequant(q, s, fmt))


def test_c_routing_and_combine_equal_numpy(libc):
    rng = np.random.default_rng(0)
    tokens, experts, top_k, hidden = 257, 19, 5, 96
    idx = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    s2s = np.zeros(tokens * top_k, dtype=np.int32)
    inv = np.zeros_like(s2s)
    counts = np.zeros(experts, dtype=np.int32)
    assert libc.mxo_routing(_p(idx), tokens * top_k, experts, _p(s2s), _p(inv), _p(counts)) == 0
    w = O.moe_init_routing(idx, experts)
    assert np.array_equal(s2s, w[0]) and np.array_equal(inv, w[1]) and np.array_equal(counts, w[2])
    bad = idx.copy(); bad[3, 1] = experts
    assert libc.mxo_routing(_p(bad), tokens * top_k, experts, _p(s2s), _p(inv), _p(counts)) == -1
    y = W.normal_bf16((tokens * top_k, hidden), 1)
    p = rng.random((tokens, top_k)).astype(np.float32)
    inv2 = w[1].copy(); inv2[7] = -1; inv2[0] = tokens * top_k
    out = np.zeros((tokens, hidden), dtype=np.uint16)
    libc.mxo_combine(_p(y), tokens * top_k, hidden, _p(inv2), _p(p), tokens, top_k, _p(out))
    assert np.array_equal(out, O.unpermute_combine(y, inv2, p))


def test_c_gemm_close_to_numpy(libc):
    rng = np.random.default_rng(2)
    aq, asc = O.mx_quant(rng.standard_normal((20, 96)).astype(np.float32))
    bq, bsc = O.mx_quant(rng.standard_normal((24, 96)).astype(np.float32))
    a, b = O.mx_dequant(aq, asc), O.mx_dequant(bq, bsc)
    c = np.zeros((20, 24), dtype=np.float32)
    libc.mxo_gemm_nt(_p(a), _p(b), 20, 24, 96, _p(c))
    assert np.allclose(c, O.mx_gemm_f32(aq, asc, bq, bsc), rtol=1e-5, atol=1e-4)


@pytest.mark.skipif(not os.path.exists(LIBREF), reason="oracle/_ref not built (reference checkout absent)")
def test_sizing_formulas_equal_reference_header():
    ref = C.CDLL(LIBREF)
    for f in (ref.ref_ub_input_quant_bytes, ref.ref_ub_dispatch_bytes, ref.ref_ub_unpermute_bytes):
        f.restype = C.c_ulonglong
    rng = np.random.default_rng(3)
    for _ in range(2000):
        m, h, k, aiv = int(rng.integers(1, 40000)), int(rng.integers(1, 20000)), int(rng.integers(1, 64)), int(rng.integers(0, 64))
        assert ref.ref_ub_input_quant_bytes(h) == O.moe_ub_input_quant_bytes(h)
        assert ref.ref_ub_dispatch_bytes(h) == O.moe_ub_dispatch_bytes(h)
        assert ref.ref_ub_unpermute_bytes(m, h, k, aiv) == O.moe_ub_unpermute_bytes(m, h, k, aiv)
        assert bool(ref.ref_ub_fits(m, h, k, aiv)) == O.moe_ub_fits(m, h, k, aiv)


@pytest.mark.skipif(not os.path.exists(REFBIN), reason="oracle/_ref not built (reference checkout absent)")
def test_reference_own_sizing_test_passes():
    r = subprocess.run([REFBIN], capture_output=True, text=True)
    assert r.returncode == 0 and "PASS" in r.stdout
