"""The oracle (CPU) and the HIP library (GPU) against vectors that the reference's own Python goldens produced.

tests/golden/make_fixtures.py ran gen_mx_quant_allgather_data.py (_quantize_fp8 with both backends, _quantize,
_quantize_to_fp4_lut, _pack_fp4_nibbles) and gen_data_moe.py (generate_dispatch_ffn_combine_mx) once, in the build
container, and wrote inputs and outputs to tests/golden/*.npz.  Nothing of the reference is needed to run these tests.
"""
import os

import numpy as np
import pytest

from oracle import mx_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
Q = np.load(os.path.join(GOLD, "quant_vectors.npz"))
F = np.load(os.path.join(GOLD, "ffn_tiny.npz"))
FINITE = slice(0, 9)          # rows of the quantizer input without Inf / NaN
NONFINITE = slice(9, 10)
BACKEND = {"lut": "lut", "native": "rne"}


# ---- CPU: oracle == golden --------------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
@pytest.mark.parametrize("backend", ["lut", "native"])
def test_oracle_fp8_quantizer_equals_the_golden(fmt, backend):
    c, s = O.mx_quant(Q["x"][FINITE], fmt, BACKEND[backend])
    assert np.array_equal(c, Q[f"fp8_{fmt}_{backend}_codes"])
    assert np.array_equal(s, Q[f"fp8_{fmt}_{backend}_scales"])
    assert np.array_equal(O.mx_dequant(c, s, fmt), Q[f"fp8_{fmt}_{backend}_dequant"])
    c, s = O.mx_quant(Q["x"][NONFINITE], fmt, BACKEND[backend])
    assert np.array_equal(c, Q[f"fp8_{fmt}_{backend}_nonfinite_codes"])
    assert np.array_equal(s, Q[f"fp8_{fmt}_{backend}_nonfinite_scales"])


@pytest.mark.parametrize("backend", ["lut", "native"])
def test_oracle_odd_block_count_pads_the_scale_row_like_the_golden(backend):
    c, s = O.mx_quant(Q["x"][FINITE, :96], "E4M3", BACKEND[backend])
    assert s.shape == (9, 4) and np.all(s[:, 3] == 127)
    assert np.array_equal(c, Q[f"fp8_E4M3_{backend}_n96_codes"])
    assert np.array_equal(s, Q[f"fp8_E4M3_{backend}_n96_scales"])


@pytest.mark.parametrize("fmt", ["E2M1", "E1M2"])
def test_oracle_fp4_quantizer_equals_the_golden(fmt):
    c, s = O.mx_quant(Q["x"][FINITE], fmt, "lut")
    assert np.array_equal(c, Q[f"fp4_{fmt}_codes"])
    assert np.array_equal(s, Q[f"fp4_{fmt}_scales"])
    assert np.array_equal(O.pack_fp4(c), Q[f"fp4_{fmt}_packed"])
    e = np.repeat(s[:, :4].astype(np.int32) - 127, 32, axis=1)
    assert np.array_equal(O.mx_dequant(c, s, fmt), np.ldexp(Q[f"fp4_{fmt}_values"], e))
    c, s = O.mx_quant(Q["x"][NONFINITE], fmt, "lut")
    assert np.array_equal(c, Q[f"fp4_{fmt}_nonfinite_codes"])
    assert np.array_equal(s, Q[f"fp4_{fmt}_nonfinite_scales"])


@pytest.mark.parametrize("fmt,fi", [("E4M3", 0), ("E5M2", 1), ("E2M1", 2)])
@pytest.mark.parametrize("backend,mi", [("native", 0), ("lut", 1)])
def test_c_oracle_quantizer_equals_the_golden(fmt, fi, backend, mi):
    """The second, independent CPU restatement (plain C) on the same vectors, non-finite row included."""
    import ctypes as C
    import subprocess
    odir = os.path.join(os.path.dirname(GOLD), "..", "oracle")
    lib_path = os.path.abspath(os.path.join(odir, "libmx_oracle.so"))
    src = os.path.abspath(os.path.join(odir, "mx_oracle.c"))
    if not os.path.exists(lib_path) or os.path.getmtime(lib_path) < os.path.getmtime(src):
        subprocess.run(["make", "-C", os.path.abspath(odir), "-B", lib_path], check=True, capture_output=True)
    lib = C.CDLL(lib_path)
    if fmt == "E2M1" and backend == "native":
        pytest.skip("the FP4 golden has the table search only")
    xb = np.ascontiguousarray(O.f32_to_bf16_bits(Q["x"][:10]))
    rows, cols = xb.shape
    codes = np.zeros((rows, cols), dtype=np.uint8)
    scales = np.zeros((rows, O.scale_cols(cols)), dtype=np.uint8)
    ptr = lambda a: a.ctypes.data_as(C.c_void_p)
    assert lib.mxo_quant_bf16(ptr(xb), rows, cols, fi, mi, ptr(codes), ptr(scales)) == 0
    if fmt == "E2M1":
        want_c = np.concatenate([Q["fp4_E2M1_codes"], Q["fp4_E2M1_nonfinite_codes"]])
        want_s = np.concatenate([Q["fp4_E2M1_scales"], Q["fp4_E2M1_nonfinite_scales"]])
    else:
        want_c = np.concatenate([Q[f"fp8_{fmt}_{backend}_codes"], Q[f"fp8_{fmt}_{backend}_nonfinite_codes"]])
        want_s = np.concatenate([Q[f"fp8_{fmt}_{backend}_scales"], Q[f"fp8_{fmt}_{backend}_nonfinite_scales"]])
    assert np.array_equal(scales, want_s)
    assert np.array_equal(codes, want_c)


def test_oracle_ffn_chain_equals_the_golden():
    """Composition of the chain: routing order, which half gets the SiLU, both bf16 roundings, nearest-even
    activations against table-rounded weights.  Every stage the golden writes out is bit-identical."""
    out, st = O.moe_ffn(F["x"], F["expert_idx"], F["gate_weight"], F["w1"], F["w1_scale"], F["w2"], F["w2_scale"], stages=True)
    assert np.array_equal(st["sorted2src"], F["sorted2src"])
    assert np.array_equal(st["y"], F["y"])                       # GMM2 output rows, expert-sorted
    # the golden combined with its CPU fallback (bf16 products, bf16 index_add_): the oracle's restatement of that
    # variant reproduces the golden's output exactly ...
    assert np.array_equal(O.unpermute_cpu_bf16(st["y"], st["sorted2src"], F["gate_weight"]), F["out"])
    # ... and the fp32 combine that the device (and this build) uses stays inside the reference's acceptance rule
    ok, err, eb = O.verify_bf16(out, O.bf16_bits_to_f32(F["out"]), int(F["shape"][1]))
    assert ok, (err, eb)


def test_ffn_vector_weights_are_what_the_table_quantizer_makes_of_their_own_dequantisation():
    """The golden stores W1 as the transpose of a [K, N] matrix quantised along K: requantising the dequantised
    rows with the table rounding must give the same bytes back (layout + idempotence)."""
    for w, ws in ((F["w1"], F["w1_scale"]), (F["w2"], F["w2_scale"])):
        for e in range(w.shape[0]):
            c, s = O.mx_quant(O.mx_dequant(w[e], ws[e]), "E4M3", "lut")
            assert np.array_equal(c, w[e]) and np.array_equal(s, ws[e])


# ---- GPU: HIP library == golden ---------------------------------------------------------------------------------
def _hip_quant(x, fmt, mode):
    import torch
    from catccos_amd import ops
    from tests.gpu_util import dev, host
    q, s = ops.mx_quant(dev(O.f32_to_bf16_bits(x)).view(torch.bfloat16), fmt, mode)
    return host(q), host(s)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
@pytest.mark.parametrize("backend", ["lut", "native"])
def test_hip_fp8_quantizer_equals_the_golden(fmt, backend):
    c, s = _hip_quant(Q["x"][FINITE], fmt, BACKEND[backend])
    assert np.array_equal(c, Q[f"fp8_{fmt}_{backend}_codes"])
    assert np.array_equal(s, Q[f"fp8_{fmt}_{backend}_scales"])
    c, s = _hip_quant(Q["x"][FINITE, :96], "E4M3", BACKEND[backend])       # general kernel, padded scale row
    assert np.array_equal(c, Q[f"fp8_E4M3_{backend}_n96_codes"]) and np.array_equal(s, Q[f"fp8_E4M3_{backend}_n96_scales"])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
@pytest.mark.parametrize("backend", ["lut", "native"])
def test_hip_fp8_quantizer_non_finite_blocks_equal_the_golden(fmt, backend):
    c, s = _hip_quant(Q["x"][NONFINITE], fmt, BACKEND[backend])
    assert np.array_equal(s, Q[f"fp8_{fmt}_{backend}_nonfinite_scales"])
    assert np.array_equal(c, Q[f"fp8_{fmt}_{backend}_nonfinite_codes"])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["E2M1", "E1M2"])
def test_hip_fp4_quantizer_equals_the_golden(fmt):
    c, s = _hip_quant(Q["x"][FINITE], fmt, "lut")
    assert np.array_equal(c, Q[f"fp4_{fmt}_packed"]) and np.array_equal(s, Q[f"fp4_{fmt}_scales"])
    c, s = _hip_quant(Q["x"][NONFINITE], fmt, "lut")
    assert np.array_equal(s, Q[f"fp4_{fmt}_nonfinite_scales"])
    assert np.array_equal(c, O.pack_fp4(Q[f"fp4_{fmt}_nonfinite_codes"]))


@pytest.mark.gpu
def test_hip_ffn_chain_on_the_golden_vector():
    """The HIP chain on the reference-made inputs: routing bit-exact, output inside the reference's acceptance rule
    and BASELINE's rtol / atol 1e-2 against the golden's own output."""
    import torch
    from catccos_amd import ops
    from tests.gpu_util import dev, host, close_bf16
    x = dev(F["x"]).view(torch.bfloat16)
    s2s, src2sorted, counts = ops.moe_init_routing(dev(F["expert_idx"]), int(F["shape"][4]))
    assert np.array_equal(host(s2s), F["sorted2src"])
    out = host(ops.dispatch_ffn_combine(x, dev(F["expert_idx"]), dev(F["gate_weight"]), dev(F["w1"]), dev(F["w1_scale"]),
                                        dev(F["w2"]), dev(F["w2_scale"])))
    gold = O.bf16_bits_to_f32(F["out"])
    ok, err, eb = O.verify_bf16(out, gold, int(F["shape"][1]))
    assert ok, (err, eb)
    bad, worst = close_bf16(out, gold, rtol=1e-2, atol=1e-2)
    assert bad == 0, (bad, worst)
