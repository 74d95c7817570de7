"""The oracle's matmul goldens, operand file layouts and FP4 packing against vectors written by the reference's own
generators of the dense MXFP8 example (gen_data_mxfp8_mmrs.py: per-element E5M2 table quantizer, [K, N] codes with
[K/64, N, 2] scales, the golden / golden_low pair) and of the FP4 grouped-matmul example
(gen_data_fp4_mx_alltoallv_gmm.py: MXFP4MatrixQuantizer, bit-level nibble packing, fp32 golden).
tests/golden/make_fixtures.py ran them once in the build container on tiny shapes; only the vectors are here.
The same files then go through the C++ driver on the GPU (-m gpu)."""
import os

import numpy as np
import pytest

from oracle import mx_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
D = np.load(os.path.join(GOLD, "mmrs_tiny.npz"))
P = np.load(os.path.join(GOLD, "fp4_gmm_tiny.npz"))
FF = np.load(os.path.join(GOLD, "ffn_tiny.npz"))


def _dense_operands():
    """K-contiguous operands from the files the example's run.sh makes (trans_a = 0, trans_b = 1)."""
    m, k, n = (int(v) for v in D["shape"])
    a, a_s = O.from_file_layout(D["tb1_a"].reshape(m, k), D["tb1_a_scale"].reshape(m, k // 64, 2), False)
    b, b_s = O.from_file_layout(D["tb1_b"].reshape(n, k), D["tb1_b_scale"].reshape(n, k // 64, 2), False)
    return m, k, n, a, a_s, b, b_s


# ---- CPU: dense MXFP8 example ---------------------------------------------------------------------------------------
def test_dense_generator_quantizer_is_the_oracle_table_quantizer():
    """The legacy per-element quantizer (nearest table value, first index on a tie) on the generator's own random
    matrices: codes and scale bytes of both operands, B quantised along its first axis."""
    m, k, n, a, a_s, b, b_s = _dense_operands()
    qa, sa = O.mx_quant(D["a_src"], "E5M2", "lut")
    qb, sb = O.mx_quant(np.ascontiguousarray(D["b_src"].T), "E5M2", "lut")
    assert np.array_equal(qa, a) and np.array_equal(sa, a_s)
    assert np.array_equal(qb, b) and np.array_equal(sb, b_s)


def test_dense_file_layouts_match_the_generator_bytes():
    """B stored [K, N] with scales [K/64, N, 2] (trans_b = 0) is to_file_layout(..., True) of the K-contiguous operand
    read from the trans_b = 1 files; A is the same bytes either way; from_file_layout inverts."""
    m, k, n, a, a_s, b, b_s = _dense_operands()
    fb, fbs = O.to_file_layout(b, b_s, True)
    assert fb.shape == (k, n) and fbs.shape == (k // 64, n, 2)
    assert np.array_equal(fb.reshape(-1), D["tb0_b"]) and np.array_equal(fbs.reshape(-1), D["tb0_b_scale"])
    fb1, fbs1 = O.to_file_layout(b, b_s, False)
    assert np.array_equal(fb1.reshape(-1), D["tb1_b"]) and np.array_equal(fbs1.reshape(-1), D["tb1_b_scale"])
    assert np.array_equal(D["tb0_a"], D["tb1_a"]) and np.array_equal(D["tb0_a_scale"], D["tb1_a_scale"])
    rb, rbs = O.from_file_layout(D["tb0_b"].reshape(k, n), D["tb0_b_scale"].reshape(k // 64, n, 2), True)
    assert np.array_equal(rb, b) and np.array_equal(rbs, b_s)


def test_dense_goldens_and_the_double_golden_rule():
    m, k, n, a, a_s, b, b_s = _dense_operands()
    gold = O.mx_gemm_f32(a, a_s, b, b_s, "E5M2", "E5M2")
    assert np.array_equal(D["tb0_golden"], D["tb1_golden"])
    assert np.allclose(gold, D["tb1_golden"], rtol=1e-5, atol=1e-5)
    # the low golden is the same product rounded to bf16: at most one unit in the last place from ours (sum order)
    low = D["tb1_golden_low"]
    ours = O.f32_to_bf16_bits(gold).astype(np.int32)
    assert np.all(np.abs(ours - low.astype(np.int32)) <= 1)
    # the rule on the generator's own pair: the low golden against the high one passes with ratios of one at most
    ok, r_max, r_mean, r_rmse, eb = O.verify_double_golden_bf16(low, D["tb1_golden"], low)
    assert ok and r_max <= 1.0 and r_mean <= 1.0 and r_rmse <= 1.0 and eb <= 2.0 ** -7
    # and an output that is off by 2 % everywhere fails it
    bad = O.f32_to_bf16_bits(D["tb1_golden"] * 1.02)
    assert not O.verify_double_golden_bf16(bad, D["tb1_golden"], low)[0]


# ---- CPU: FP4 grouped-matmul example --------------------------------------------------------------------------------
def _fp4_operands():
    m, k, n, e = (int(v) for v in P["shape"])
    a = O.unpack_fp4(P["input_a"].reshape(m, k // 2))
    a_s = P["input_a_scale"].reshape(m, k // 32)
    fb = P["input_b"].reshape(e, k, n // 2)                       # [K, N] codes, pairs along N
    fbs = P["input_b_scale"].reshape(e, k // 64, n, 2)
    b = np.stack([np.ascontiguousarray(O.unpack_fp4(fb[i]).T) for i in range(e)])                     # [E, N, K]
    b_s = np.stack([fbs[i].transpose(1, 0, 2).reshape(n, k // 32) for i in range(e)])
    return m, k, n, e, a, a_s, b, b_s


def test_fp4_generator_quantizer_and_packing_are_the_oracle_ones():
    m, k, n, e, a, a_s, b, b_s = _fp4_operands()
    qa, sa = O.mx_quant(P["a_src"], "E2M1", "lut")
    assert np.array_equal(qa, a) and np.array_equal(sa, a_s)
    assert np.array_equal(O.pack_fp4(qa).reshape(-1), P["input_a"])
    for i in range(e):
        qb, sb = O.mx_quant(np.ascontiguousarray(P["b_src"][i].T), "E2M1", "lut")
        assert np.array_equal(qb, b[i]) and np.array_equal(sb, b_s[i]), i
        fb, fbs = O.to_file_layout_fp4(qb, sb, True)
        assert np.array_equal(fb.reshape(-1), P["input_b"].reshape(e, -1)[i])
        assert np.array_equal(fbs.reshape(-1), P["input_b_scale"].reshape(e, -1)[i])
    fa, fas = O.to_file_layout_fp4(qa, sa, False)
    assert np.array_equal(fa.reshape(-1), P["input_a"]) and np.array_equal(fas.reshape(-1), P["input_a_scale"])


def test_fp4_grouped_golden():
    m, k, n, e, a, a_s, b, b_s = _fp4_operands()
    counts = P["local_tokens_per_expert"]
    assert counts.sum() == m and np.array_equal(counts, P["global_tokens_per_local_expert"])
    gold = O.mx_gmm_f32(a, a_s, b, b_s, counts, "E2M1", "E2M1")
    assert np.allclose(gold, P["golden"], rtol=1e-5, atol=1e-4)


# ---- GPU: the same files through the C++ driver ------------------------------------------------------------------------
from tests.test_host_layer import host_bin, _run          # noqa: E402,F401  (the driver's fixture and launcher)


@pytest.mark.gpu
@pytest.mark.parametrize("trans_b", [1, 0])
def test_driver_dense_on_the_generator_files(host_bin, tmp_path, trans_b):
    """rank_0_{a,b,a_scale,b_scale}.bin exactly as gen_data_mxfp8_mmrs.py wrote them -> output.bin judged by the
    example's own double-golden rule against its golden.bin / golden_low.bin."""
    m, k, n = (int(v) for v in D["shape"])
    for what in ("a", "b", "a_scale", "b_scale"):
        D[f"tb{trans_b}_{what}"].tofile(tmp_path / f"rank_0_{what}.bin")
    r = _run(host_bin, "Ascend950MxFp8MatmulReduceScatter", m, k, n, "--data", tmp_path, "--fmt", "e5m2", "--transa", 0,
             "--transb", trans_b, "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output.bin", dtype=np.uint16).reshape(m, n)
    gold, low = D[f"tb{trans_b}_golden"], D[f"tb{trans_b}_golden_low"]
    ok, r_max, r_mean, r_rmse, eb = O.verify_double_golden_bf16(got, gold, low)
    assert ok, (r_max, r_mean, r_rmse, eb)
    assert np.allclose(O.bf16_bits_to_f32(got), gold, rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
def test_driver_fp4_grouped_on_the_generator_files(host_bin, tmp_path):
    m, k, n, e = (int(v) for v in P["shape"])
    for stem in ("input_a", "input_a_scale", "input_b", "input_b_scale", "local_tokens_per_expert", "global_tokens_per_local_expert"):
        P[stem].tofile(tmp_path / f"{stem}_0.bin")
    r = _run(host_bin, "Ascend950Fp4MxAllToAllVGroupedMatmul", m, k, n, "--experts", e, "--data", tmp_path, "--transb", 0, "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output_0.bin", dtype=np.float16).reshape(m, n).astype(np.float32)
    gold = P["golden"]
    # the example's acceptance (verify_result.py with an fp16 output, K < 2048): every element within 2^-8 * max(1, |gold|)
    assert np.all(np.abs(got - gold) <= 2.0 ** -8 * np.maximum(1.0, np.abs(gold)))


@pytest.mark.gpu
def test_driver_ffn_on_the_generator_files(host_bin, tmp_path):
    """The seven input files of generate_dispatch_ffn_combine_mx -> output_0.bin judged by verify_result.py's bf16 rule
    against out_gather_combine_0.bin."""
    m, k, n, top_k, e = (int(v) for v in FF["shape"])
    for stem, key in (("in_routing_matrix_a", "x"), ("in_gmm_matrix_b", "w1"), ("in_gmm_matrix_b_scale", "w1_scale"),
                      ("in_gmm_matrix_b2", "w2"), ("in_gmm_matrix_b2_scale", "w2_scale"), ("in_routing_expert_idx", "expert_idx"),
                      ("in_gather_gate_weight", "gate_weight")):
        np.ascontiguousarray(FF[key]).tofile(tmp_path / f"{stem}_0.bin")
    r = _run(host_bin, "Ascend950DispatchFFNCombine", m, k, n, "--experts", e, "--topk", top_k, "--data", tmp_path, "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output_0.bin", dtype=np.uint16).reshape(m, k)
    ok, err, eb = O.verify_bf16(got, O.bf16_bits_to_f32(FF["out"]), k)
    assert ok, (err, eb)
