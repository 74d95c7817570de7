"""INT8 W8A8 path: per-token quantise + scatter (bit-exact), grouped matmul + dequant + SwiGLU (INT32 sums exact, fp16
step exact, sigmoid within a few ulp: rtol 1e-5 on the fp32 output)."""
import numpy as np
import pytest
import torch

from oracle import int8_oracle as Q
from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import dev, host, bf16_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,k,top_k", [(5, 64, 1), (33, 7168, 4), (16, 264, 3), (300, 2048, 8)])
def test_quant_scatter_bit_exact(tokens, k, top_k):
    from catccos_amd import ops
    xb = W.activations_with_outliers(tokens, k, seed=tokens + k)
    xb[tokens // 2] = 0                                            # a row of zeros
    rng = np.random.default_rng(k)
    idx = rng.integers(0, 6, size=(tokens, top_k)).astype(np.int32)
    sorted2src = np.argsort(idx.reshape(-1), kind="stable").astype(np.int32)
    src2sorted = np.empty_like(sorted2src)
    src2sorted[sorted2src] = np.arange(sorted2src.size, dtype=np.int32)
    codes, scales = ops.int8_quant_scatter(bf16_dev(xb), dev(src2sorted), top_k)
    wq, ws = Q.dispatch_quant(O.bf16_bits_to_f32(xb), sorted2src, top_k)
    assert np.array_equal(host(codes), wq)
    assert np.array_equal(host(scales), ws)


def _case(rng, counts, n, k, lo=-16, hi=16):
    e = len(counts)
    rows = sum(counts)
    a = rng.integers(lo, hi, size=(rows, k), dtype=np.int8)
    b = rng.integers(lo, hi, size=(e, k, n), dtype=np.int8)
    ch = Q.truncate_scale(rng.standard_normal(e * n).astype(np.float32) / 127)
    ts = (np.abs(rng.standard_normal(rows)) / 127 + 1e-3).astype(np.float32)
    return a, ts, b, ch


@pytest.mark.parametrize("counts,n,k", [([5, 0, 300, 1, 0, 257, 64], 256, 256), ([512], 1024, 7168), ([0, 0, 7], 64, 128),
                                        ([1] * 9, 320, 384), ([256, 256], 512, 1024)])
@pytest.mark.parametrize("trans_b", [0, 1])
def test_gmm_dequant_swiglu_vs_oracle(counts, n, k, trans_b):
    from catccos_amd import ops
    rng = np.random.default_rng(sum(counts) + n + k)
    a, ts, b, ch = _case(rng, counts, n, k)
    bd = dev(np.ascontiguousarray(b.transpose(0, 2, 1))) if trans_b else dev(b)
    out = ops.int8_gmm_dequant_swiglu(dev(a), dev(ts), bd, dev(ch), dev(np.array(counts, dtype=np.int32)), n, k, trans_b)
    gold = Q.gmm_dequant_swiglu(a, ts, b, ch, counts)
    got = host(out)
    assert np.allclose(got, gold, rtol=1e-5, atol=1e-7), np.abs(got - gold).max()


def test_full_range_codes_and_scale_words():
    """Codes over the whole int8 range at K = 7168 (sums up to 2^27), scales read from the reference's file format
    (64-bit words, fp32 in the low half), fp16 and bf16 outputs, rows past the groups untouched."""
    from catccos_amd import ops
    rng = np.random.default_rng(9)
    counts = [130, 70]
    n, k = 256, 7168
    a, ts, b, _ = _case(rng, counts, n, k, -128, 128)
    ch = Q.truncate_scale(rng.standard_normal(2 * n).astype(np.float32) * 1e-4)      # keeps fp16(c * scale) finite
    words = torch.from_numpy(Q.channel_scale_words(ch)).cuda()
    rows = sum(counts)
    a_pad = np.concatenate([a, np.zeros((6, k), dtype=np.int8)])
    ts_pad = np.concatenate([ts, np.ones(6, dtype=np.float32)])
    gold = Q.gmm_dequant_swiglu(a, ts, b, ch, counts)
    for out, rt in (("fp32", 1e-5), ("fp16", 2e-3), ("bf16", 1e-2)):
        c = torch.full((rows + 6, n // 2), 7.0, dtype={"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}[out],
                       device="cuda")
        ops.int8_gmm_dequant_swiglu(dev(a_pad), dev(ts_pad), dev(b), words.view(torch.float32), dev(np.array(counts, dtype=np.int32)),
                                    n, k, 0, out, scale_stride=2, c=c)
        got = c.float().cpu().numpy()
        assert np.allclose(got[:rows], gold, rtol=rt, atol=1e-6 if out == "fp32" else 1e-3), (out, np.abs(got[:rows] - gold).max())
        assert np.all(got[rows:] == 7.0)


def test_int32_sums_are_exact():
    """Unit scales and a gate column pinned to 1: the output is silu(c) for integer c, exact wherever fp16 holds c."""
    from catccos_amd import ops
    rng = np.random.default_rng(4)
    k, n = 128, 64
    a = rng.integers(-3, 4, size=(64, k), dtype=np.int8)
    b = np.zeros((1, k, n), dtype=np.int8)
    b[0, :, :32] = rng.integers(-3, 4, size=(k, 32), dtype=np.int8)
    b[0, 0, 32:] = 1
    a[:, 0] = 1                                                     # gate = 1 * 1 = 1
    c = a.astype(np.int32) @ b[0].astype(np.int32)
    assert np.abs(c).max() < 2048 and np.all(c[:, 32:] == 1)
    out = host(ops.int8_gmm_dequant_swiglu(dev(a), dev(np.ones(64, dtype=np.float32)), dev(b), dev(np.ones(n, dtype=np.float32)),
                                           dev(np.array([64], dtype=np.int32)), n, k))
    x0 = c[:, :32].astype(np.float64)
    assert np.allclose(out, x0 / (1 + np.exp(-x0)), rtol=1e-5, atol=1e-30)
    assert np.array_equal(out[c[:, :32] == 0], np.zeros(np.count_nonzero(c[:, :32] == 0), dtype=np.float32))


def test_bad_arguments():
    from catccos_amd import _lib
    lib = _lib.load()
    z = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    assert lib.cmx_int8_gmm_dequant_swiglu(p, 128, p, p, p, 1, p, 32, 2, p, 1, 4, 64, 96, 1, p, None) == -1     # k % 128
    assert lib.cmx_int8_gmm_dequant_swiglu(p, 128, p, p, p, 1, p, 32, 2, p, 1, 4, 48, 128, 1, p, None) == -1    # n % 64
    assert lib.cmx_int8_gmm_dequant_swiglu(p, 128, p, p, p, 0, p, 32, 2, p, 1, 4, 64, 128, 1, p, None) == -1    # stride
    assert lib.cmx_int8_quant_scatter(p, 64, None, p, 64, p, 4, 64, 2, None) == -1                            # no table, top_k 2
