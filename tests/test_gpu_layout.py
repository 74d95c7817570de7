"""Operands stored with K as the slow axis ([K, N] codes, [K/64, N, 2] scales): the layout kernel is pure
data movement and must be bit-exact; the matmul entry points that accept either orientation must give the
same bits as the K-contiguous ones."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from tests.gpu_util import dev, host, close_bf16

pytestmark = pytest.mark.gpu


def _mx(rng, rows, k, fmt="E4M3"):
    return O.mx_quant(O.bf16_round(rng.standard_normal((rows, k)).astype(np.float32)), fmt)


@pytest.mark.parametrize("n,k", [(128, 128), (1, 64), (37, 192), (130, 320), (4096, 7168), (257, 64), (64, 1024)])
def test_to_k_major_is_bit_exact(n, k):
    from catccos_amd import ops
    rng = np.random.default_rng(n + k)
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    scales = rng.integers(0, 256, size=(n, k // 32), dtype=np.uint8)
    fc, fs = O.to_file_layout(codes, scales, True)
    d, ds = ops.mx_to_k_major(dev(fc), dev(fs), k, n)
    assert np.array_equal(host(d), codes)
    assert np.array_equal(host(ds), scales)


def test_to_k_major_batched_and_unaligned_source():
    from catccos_amd import ops, _lib
    rng = np.random.default_rng(5)
    g, n, k = 5, 70, 256
    codes = rng.integers(0, 256, size=(g, n, k), dtype=np.uint8)
    scales = rng.integers(0, 256, size=(g, n, k // 32), dtype=np.uint8)
    fc = np.stack([O.to_file_layout(codes[i], scales[i], True)[0] for i in range(g)])
    fs = np.stack([O.to_file_layout(codes[i], scales[i], True)[1] for i in range(g)])
    d, ds = ops.mx_to_k_major(dev(fc), dev(fs), k, n)
    assert np.array_equal(host(d), codes) and np.array_equal(host(ds), scales)
    # a source whose rows are not dword aligned (n = 70 starting one byte in) and padded destination pitches
    lib = _lib.load()
    src = torch.zeros(k * n + 1, dtype=torch.uint8, device="cuda")
    src[1:] = dev(fc[0]).reshape(-1)
    dst = torch.full((n, k + 16), 0xAA, dtype=torch.uint8, device="cuda")
    dsc = torch.full((n, k // 32 + 3), 0xBB, dtype=torch.uint8, device="cuda")
    _lib.check(lib.cmx_mx_to_k_major(src.data_ptr() + 1, n, dev(fs[0]).data_ptr(), dst.data_ptr(), k + 16, dsc.data_ptr(),
                                     k // 32 + 3, k, n, 1, torch.cuda.current_stream().cuda_stream))
    assert np.array_equal(host(dst)[:, :k], codes[0]) and np.all(host(dst)[:, k:] == 0xAA)
    assert np.array_equal(host(dsc)[:, :k // 32], scales[0]) and np.all(host(dsc)[:, k // 32:] == 0xBB)


@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
@pytest.mark.parametrize("trans_a,trans_b", [(0, 0), (1, 1), (1, 0), (0, 1)])
def test_gemm_ex_matches_the_k_contiguous_entry_point(fmt, trans_a, trans_b):
    from catccos_amd import ops
    rng = np.random.default_rng(17 + trans_a * 2 + trans_b)
    m, n, k = 200, 300, 512
    aq, asc = _mx(rng, m, k, fmt)
    bq, bsc = _mx(rng, n, k, fmt)
    fa, fas = O.to_file_layout(aq, asc, bool(trans_a))
    fb, fbs = O.to_file_layout(bq, bsc, not trans_b)
    c = ops.mx_gemm_ex(dev(fa), dev(fas), dev(fb), dev(fbs), m, n, k, fmt, "bf16", trans_a, trans_b)
    ref = ops.mx_gemm(dev(aq), dev(asc[:, :k // 32].copy()), dev(bq), dev(bsc[:, :k // 32].copy()), k, fmt, "bf16")
    assert np.array_equal(host(c), host(ref))
    bad, worst = close_bf16(host(c), O.mx_gemm_f32(aq, asc, bq, bsc, fmt, fmt))
    assert bad == 0, (bad, worst)


def test_gmm_ex_with_k_slow_weights():
    from catccos_amd import ops
    rng = np.random.default_rng(23)
    counts = [70, 0, 300, 3]
    n, k = 192, 256
    m = sum(counts)
    aq, asc = _mx(rng, m, k)
    ws_ = [_mx(rng, n, k) for _ in counts]
    wq, wsc = np.stack([q for q, _ in ws_]), np.stack([s for _, s in ws_])
    fw = np.stack([O.to_file_layout(wq[i], wsc[i], True)[0] for i in range(len(counts))])
    fws = np.stack([O.to_file_layout(wq[i], wsc[i], True)[1] for i in range(len(counts))])
    gs = dev(np.array(counts, dtype=np.int32))
    c0 = ops.mx_gmm_ex(dev(aq), dev(asc), dev(fw), dev(fws), gs, n, k, trans_b=0)
    c1 = ops.mx_gmm_ex(dev(aq), dev(asc), dev(wq), dev(wsc), gs, n, k, trans_b=1)
    assert np.array_equal(host(c0), host(c1))
    bad, worst = close_bf16(host(c0), O.mx_gmm_f32(aq, asc, wq, wsc, counts))
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("n,k", [(128, 128), (2, 64), (37, 192), (130, 320), (4096, 7168), (255, 64), (64, 1024)])
def test_fp4_to_k_major_is_bit_exact(n, k):
    from catccos_amd import ops
    rng = np.random.default_rng(n * 3 + k)
    codes = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    scales = rng.integers(0, 256, size=(n, k // 32), dtype=np.uint8)
    fb, fs = O.to_file_layout_fp4(codes, scales, True)
    d, ds = ops.mxfp4_to_k_major(dev(fb), dev(fs), k, n)
    assert np.array_equal(host(d), O.pack_fp4(codes))
    assert np.array_equal(host(ds), scales)


def test_fp4_batched_weights_and_grouped_matmul_ex():
    from catccos_amd import ops
    rng = np.random.default_rng(29)
    counts = [40, 0, 129, 300]
    n, k = 256, 512
    m = sum(counts)
    aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
    ws_ = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in counts]
    wq, wsc = np.stack([q for q, _ in ws_]), np.stack([s_ for _, s_ in ws_])
    fw = np.stack([O.to_file_layout_fp4(wq[i], wsc[i], True)[0] for i in range(len(counts))])
    fws = np.stack([O.to_file_layout_fp4(wq[i], wsc[i], True)[1] for i in range(len(counts))])
    d, ds = ops.mxfp4_to_k_major(dev(fw), dev(fws), k, n)
    assert np.array_equal(host(d), np.stack([O.pack_fp4(w) for w in wq])) and np.array_equal(host(ds), wsc)
    gs = dev(np.array(counts, dtype=np.int32))
    c0 = ops.mx_gmm_ex(dev(O.pack_fp4(aq)), dev(asc), dev(fw), dev(fws), gs, n, k, "E2M1", "fp16", trans_b=0)
    c1 = ops.mx_gmm(dev(O.pack_fp4(aq)), dev(asc), dev(O.pack_fp4(wq)), dev(wsc), gs, k, "E2M1", "fp16")
    assert np.array_equal(host(c0), host(c1))
    gold = O.mx_gmm_f32(aq, asc, wq, wsc, counts, "E2M1", "E2M1")
    assert np.allclose(host(c0).astype(np.float64), gold, rtol=2e-3, atol=5e-2)


def test_fp4_gemm_ex_orientations():
    from catccos_amd import ops
    rng = np.random.default_rng(30)
    m, n, k = 130, 300, 640
    aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
    bq, bsc = O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1")
    ref = ops.mx_gemm(dev(O.pack_fp4(aq)), dev(asc), dev(O.pack_fp4(bq)), dev(bsc), k, "E2M1", "fp32")
    for trans_a, trans_b in [(0, 0), (1, 1), (1, 0)]:
        fa, fas = O.to_file_layout_fp4(aq, asc, bool(trans_a))
        fb, fbs = O.to_file_layout_fp4(bq, bsc, not trans_b)
        c = ops.mx_gemm_ex(dev(fa), dev(fas), dev(fb), dev(fbs), m, n, k, "E2M1", "fp32", trans_a, trans_b)
        assert np.array_equal(host(c), host(ref)), (trans_a, trans_b)
    assert np.allclose(host(ref), O.mx_gemm_f32(aq, asc, bq, bsc, "E2M1", "E2M1"), rtol=1e-5, atol=1e-3)


def test_ex_entry_points_reject_what_they_do_not_cover():
    from catccos_amd import _lib
    lib = _lib.load()
    z = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    assert lib.cmx_mx_gemm_ex(p, p, p, p, p, 64, 64, 64, 64, 3, 0, 0, 0, p, None) == -1      # E1M2 has no matmul
    assert lib.cmx_mx_gemm_ex(p, p, p, p, p, 64, 64, 64, 96, 0, 0, 0, 0, p, None) == -1      # k % 64
    assert lib.cmx_mx_gemm_ex(p, p, p, p, p, 64, 64, 64, 64, 0, 0, 0, 0, None, None) == -1   # workspace missing
    assert lib.cmx_mx_gemm_ex_workspace_bytes(64, 64, 64, 0, 1) == 0
