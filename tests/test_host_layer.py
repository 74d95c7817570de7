"""The C++ plugin layer (CatccosOperator / OperatorRegistry / launch table / driver).

CPU part: the host-only C++ check program and the driver's argument and validation paths, none of
which reach the GPU.  GPU part: the driver end to end on .bin files written from seeded inputs, its
output files compared with the oracle the same way the library-level parity tests do.
"""
import os
import subprocess

import numpy as np
import pytest

from oracle import mx_oracle as O
from catccos_amd import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "catccos_amd", "host")
BIN = os.path.join(HOST, "bin")


@pytest.fixture(scope="module")
def host_bin():
    if not (os.path.exists(os.path.join(BIN, "catccos_mx_run")) and os.path.exists(os.path.join(BIN, "test_host_layer"))):
        from catccos_amd import build
        build.build(force=False)
        subprocess.run(["make", "-C", HOST, "all"], check=True, capture_output=True)
    return BIN


def _run(host_bin, *args, timeout=120):
    return subprocess.run([os.path.join(host_bin, "catccos_mx_run"), *map(str, args)], capture_output=True, text=True, timeout=timeout)


def test_host_checks(host_bin):
    r = subprocess.run([os.path.join(host_bin, "test_host_layer")], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host layer checks: PASS" in r.stdout


def test_driver_rejects_before_touching_the_gpu(host_bin):
    r = _run(host_bin, "a5moe", 4, 7168)
    assert r.returncode == 1 and "Usage" in r.stderr
    r = _run(host_bin, "NoSuchOperator", 4, 256, 512)
    assert r.returncode != 0 and "not found" in r.stdout
    r = _run(host_bin, "a5moe", 4, 7168 + 128, 4096)                   # K % 256 != 0
    assert r.returncode != 0 and "Invalid CocTilingParams" in r.stderr
    r = _run(host_bin, "a5moe", 4, 7168, 4096, "--experts", 4, "--topk", 6)      # topK > experts
    assert r.returncode != 0 and "Invalid CocTilingParams" in r.stderr
    r = _run(host_bin, "a5moe", 0, 7168, 4096)
    assert r.returncode == 1 and "positive uint32" in r.stderr
    r = _run(host_bin, "a5moe", 4, 7168, 4096, "--m0", 64)
    assert r.returncode == 1 and "Invalid GMM1 M tile" in r.stderr
    r = _run(host_bin, "mxqtag", 16, 1, 7168 + 16)                      # columns not a multiple of 32
    assert r.returncode != 0


# ---------------------------------------------------------------------------------------------- GPU

def _write(path, arr):
    np.ascontiguousarray(arr).tofile(path)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,ofmt", [("e4m3", "E4M3"), ("e5m2", "E5M2"), ("e2m1", "E2M1"), ("e1m2", "E1M2")])
def test_driver_quant(host_bin, tmp_path, fmt, ofmt):
    rows, cols = 96, 7168
    x = W.activations_with_outliers(rows, cols, seed=5)
    _write(tmp_path / "rank_0_input.bin", x)
    r = _run(host_bin, "MxQuantAllGather", rows, 1, cols, "--data", tmp_path, "--fmt", fmt, "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "[TEST] input rank_size: 1 rank_id:0" in r.stdout and "[CONFIG]" in r.stdout
    fp4 = ofmt in ("E2M1", "E1M2")
    codes, scales = O.mx_quant_bf16(x, ofmt, "lut" if fp4 else "rne")
    if fp4:
        codes = O.pack_fp4(codes)
    got = np.fromfile(tmp_path / "rank_0_output.bin", dtype=np.uint8).reshape(codes.shape)
    got_s = np.fromfile(tmp_path / "rank_0_mxscale.bin", dtype=np.uint8).reshape(scales.shape)
    assert np.array_equal(got, codes) and np.array_equal(got_s, scales)


@pytest.mark.gpu
def test_driver_quant_odd_block_count_writes_unpadded_scale_rows(host_bin, tmp_path):
    """N = 96: the reference operator writes exactly N / 32 = 3 scale bytes per row (mx_quant_allgather_host.h:47-87)."""
    rows, cols = 40, 96
    x = W.activations_with_outliers(rows, cols, seed=6)
    _write(tmp_path / "rank_0_input.bin", x)
    r = _run(host_bin, "MxQuantAllGather", rows, 1, cols, "--data", tmp_path, "--fmt", "e4m3", "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    codes, scales = O.mx_quant_bf16(x, "E4M3", "rne")
    assert np.array_equal(np.fromfile(tmp_path / "rank_0_output.bin", dtype=np.uint8).reshape(rows, cols), codes)
    assert np.array_equal(np.fromfile(tmp_path / "rank_0_mxscale.bin", dtype=np.uint8).reshape(rows, 3), scales[:, :3])


@pytest.mark.gpu
def test_driver_mxfp8_matmul(host_bin, tmp_path):
    m, k, n = 192, 1024, 384
    rng = np.random.default_rng(11)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)), "E4M3", "rne")
    bq, bsc = O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut")
    for stem, arr in (("a", aq), ("b", bq), ("a_scale", asc), ("b_scale", bsc)):
        _write(tmp_path / f"rank_0_{stem}.bin", arr)
    r = _run(host_bin, "a5mxfp8mmrs", m, k, n, "--data", tmp_path)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output.bin", dtype=np.uint16).reshape(m, n)
    gold = O.mx_gemm_f32(aq, asc, bq, bsc)
    assert np.allclose(O.bf16_bits_to_f32(got), gold, rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("trans_a,trans_b", [(0, 0), (1, 0), (1, 1)])
def test_driver_mxfp8_matmul_operand_orientations(host_bin, tmp_path, trans_a, trans_b):
    """Input files in the generator's other orientations (gen_data_mxfp8_mmrs.py:309-330), E5M2 as in the
    reference example's main.cpp:20-21."""
    m, k, n = 160, 512, 320
    rng = np.random.default_rng(13)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)), "E5M2", "rne")
    bq, bsc = O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E5M2", "rne")
    fa, fas = O.to_file_layout(aq, asc, bool(trans_a))
    fb, fbs = O.to_file_layout(bq, bsc, not trans_b)
    for stem, arr in (("a", fa), ("b", fb), ("a_scale", fas), ("b_scale", fbs)):
        _write(tmp_path / f"rank_0_{stem}.bin", arr)
    r = _run(host_bin, "a5mxfp8mmrs", m, k, n, "--data", tmp_path, "--fmt", "e5m2", "--transa", trans_a, "--transb", trans_b,
             "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output.bin", dtype=np.uint16).reshape(m, n)
    gold = O.mx_gemm_f32(aq, asc, bq, bsc, "E5M2", "E5M2")
    assert np.allclose(O.bf16_bits_to_f32(got), gold, rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("trans_b", [0, 1])
def test_driver_fp4_grouped_matmul(host_bin, tmp_path, trans_b):
    """The reference's file names and both weight orientations of its generator (transB = 0 is its run.sh default:
    examples/ascend950_fp4_mx_alltoallv_grouped_matmul/scripts/run.sh:16-17)."""
    experts, n, k = 4, 192, 256
    counts = np.array([40, 0, 70, 18], dtype=np.int32)
    m = int(counts.sum())
    rng = np.random.default_rng(19)
    aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
    ws_ = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in range(experts)]
    wq, wsc = np.stack([q for q, _ in ws_]), np.stack([s_ for _, s_ in ws_])
    fb = np.stack([O.to_file_layout_fp4(wq[i], wsc[i], not trans_b)[0] for i in range(experts)])
    fbs = np.stack([O.to_file_layout_fp4(wq[i], wsc[i], not trans_b)[1] for i in range(experts)])
    fa, fas = O.to_file_layout_fp4(aq, asc, False)
    for stem, arr in (("input_a", fa), ("input_a_scale", fas), ("input_b", fb), ("input_b_scale", fbs),
                      ("local_tokens_per_expert", counts), ("global_tokens_per_local_expert", counts)):
        _write(tmp_path / f"{stem}_0.bin", arr)
    r = _run(host_bin, "a5fp4mxatavgmm", m, k, n, "--experts", experts, "--data", tmp_path, "--transb", trans_b, "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output_0.bin", dtype=np.float16).reshape(m, n).astype(np.float64)
    gold = O.mx_gmm_f32(aq, asc, wq, wsc, counts, "E2M1", "E2M1")
    assert np.allclose(got, gold, rtol=2e-3, atol=5e-2)


FAMILY = [   # short name, fp4, grouped, file name style, output file
    ("a5fp8mxagmm", False, False, "input", "output_0.bin"),
    ("a5fp4mxagmm", True, False, "input", "output_0.bin"),
    ("a5mxfp8mmata", False, False, "rank", "output_0.bin"),
    ("a5fp4mmrs", True, False, "rank", "output.bin"),
    ("a5mxfp8atammsplitkurma", False, False, "input", "output_0.bin"),
    ("a5fp8mxatavgmm", False, True, "input", "output_0.bin"),
    ("a5fp8gmmata", False, True, "gm", "output_0.bin"),
    ("a5fp4gmmata", True, True, "gm", "output_0.bin"),
]


@pytest.mark.gpu
@pytest.mark.parametrize("short,fp4,grouped,style,outfile", FAMILY)
def test_driver_mx_matmul_family(host_bin, tmp_path, short, fp4, grouped, style, outfile):
    """The other MX matmul operators of the reference under their own names, file names and default orientation
    (transB = 0: weights [K, N] with scales [K/64, N, 2]); fp16 output."""
    fmt = "E2M1" if fp4 else "E4M3"
    experts, n, k = (4 if grouped else 1), 192, 256
    counts = np.array([40, 0, 70, 18], dtype=np.int32) if grouped else np.array([96], dtype=np.int32)
    m = int(counts.sum())
    rng = np.random.default_rng(len(short) + 7 * fp4)
    gen = (lambda r: rng.uniform(-2, 2, (r, k)).astype(np.float32)) if fp4 else \
          (lambda r: O.bf16_round(rng.standard_normal((r, k)).astype(np.float32)))
    aq, asc = O.mx_quant(gen(m), fmt)
    ws_ = [O.mx_quant(gen(n), fmt) for _ in range(experts)]
    wq, wsc = np.stack([q for q, _ in ws_]), np.stack([s_ for _, s_ in ws_])
    lay = O.to_file_layout_fp4 if fp4 else O.to_file_layout
    fb = np.stack([lay(wq[i], wsc[i], True)[0] for i in range(experts)])
    fbs = np.stack([lay(wq[i], wsc[i], True)[1] for i in range(experts)])
    fa, fas = lay(aq, asc, False)
    name = {"input": lambda w: f"input_{w}_0.bin", "rank": lambda w: f"rank_0_{w}.bin",
            "gm": lambda w: (f"{w}_gm_0.bin" if w in ("a", "b") else f"{w}_0.bin")}[style]
    for what, arr in (("a", fa), ("b", fb), ("a_scale", fas), ("b_scale", fbs)):
        _write(tmp_path / name(what), arr)
    args = [short, m, k, n, "--data", tmp_path, "--transb", 0, "--poison"]
    if grouped:
        _write(tmp_path / "local_tokens_per_expert_0.bin", counts)
        _write(tmp_path / "global_tokens_per_local_expert_0.bin", counts)
        args += ["--experts", experts]
    r = _run(host_bin, *args)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / outfile, dtype=np.float16).reshape(m, n).astype(np.float64)
    gold = O.mx_gmm_f32(aq, asc, wq, wsc, counts, fmt, fmt)
    assert np.allclose(got, gold, rtol=2e-3, atol=5e-2)


@pytest.mark.gpu
def test_driver_int8_dispatch_gmm_dequant_swiglu(host_bin, tmp_path):
    """The reference operator's own arithmetic and file names (examples/dispatch_gmm_dequant_swiglu/
    dispatch_gmm_dequant_swiglu_host.h:31-73): a_gm bf16 [m, k], b_gm int8 [E, k, n], scale_gm 64-bit words,
    expert_idx int32 [m, topK] -> output bf16 [m * topK, n / 2], rows sorted by expert."""
    from oracle import int8_oracle as Q
    m, k, n, experts, top_k = 48, 512, 256, 4, 4
    rng = np.random.default_rng(31)
    x = W.normal_bf16((m, k), 6)
    idx = rng.integers(0, experts, size=(m, top_k)).astype(np.int32)
    b = rng.integers(-16, 16, size=(experts, k, n), dtype=np.int8)
    ch = Q.truncate_scale(rng.standard_normal(experts * n).astype(np.float32) / 127)
    for stem, arr in (("a_gm", x), ("b_gm", b), ("scale_gm", Q.channel_scale_words(ch)), ("expert_idx", idx)):
        _write(tmp_path / f"{stem}_0.bin", arr)
    r = _run(host_bin, "DispatchGmmDequantSwiglu", m, k, n, "--experts", experts, "--topk", top_k, "--data", tmp_path,
             "--arith", "int8", "--poison")
    assert r.returncode == 0, r.stdout + r.stderr
    sorted2src = np.argsort(idx.reshape(-1), kind="stable")
    counts = np.bincount(idx.reshape(-1), minlength=experts)
    aq, ts = Q.dispatch_quant(O.bf16_bits_to_f32(x), sorted2src, top_k)
    gold = Q.gmm_dequant_swiglu(aq, ts, b, ch, counts)
    got = O.bf16_bits_to_f32(np.fromfile(tmp_path / "output_0.bin", dtype=np.uint16).reshape(m * top_k, n // 2))
    assert np.allclose(got, gold, rtol=1e-2, atol=1e-3)


@pytest.mark.gpu
def test_driver_ffn(host_bin, tmp_path):
    tokens, k, n, experts, top_k = 64, 512, 1024, 8, 4
    rng = np.random.default_rng(3)
    x = W.normal_bf16((tokens, k), 3)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, 4)
    w1 = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut") for _ in range(experts)]
    w2 = [O.mx_quant(O.bf16_round(rng.standard_normal((k, n // 2)).astype(np.float32) / np.sqrt(n // 2)), "E4M3", "lut") for _ in range(experts)]
    w1q, w1s = np.stack([a for a, _ in w1]), np.stack([b for _, b in w1])
    w2q, w2s = np.stack([a for a, _ in w2]), np.stack([b for _, b in w2])
    for stem, arr in (("in_routing_matrix_a", x), ("in_gmm_matrix_b", w1q), ("in_gmm_matrix_b2", w2q), ("in_gmm_matrix_b_scale", w1s),
                      ("in_gmm_matrix_b2_scale", w2s), ("in_routing_expert_idx", idx.astype(np.int32)), ("in_gather_gate_weight", p.astype(np.float32))):
        _write(tmp_path / f"{stem}_0.bin", arr)
    r = _run(host_bin, "Ascend950DispatchFFNCombine", tokens, k, n, "--experts", experts, "--topk", top_k, "--data", tmp_path, "--poison",
             "--repeats", 2)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(tmp_path / "output_0.bin", dtype=np.uint16).reshape(tokens, k)
    gold = O.bf16_bits_to_f32(O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s))
    ok, err, eb = O.verify_bf16(got, gold, 1 << 20)
    diff = np.abs(O.bf16_bits_to_f32(got) - gold)
    assert (diff > 1e-2 + 1e-2 * np.abs(gold)).sum() <= got.size // 1000 and eb <= 2.0 ** -7, (err, eb)
    # a missing input file is an error, not a silent default
    os.remove(tmp_path / "in_gather_gate_weight_0.bin")
    r = _run(host_bin, "a5moe", tokens, k, n, "--experts", experts, "--topk", top_k, "--data", tmp_path)
    assert r.returncode != 0 and "ERROR" in r.stderr
