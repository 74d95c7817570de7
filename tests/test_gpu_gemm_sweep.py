"""Seeded shape sweep of the dense and grouped matmuls under the default tile heuristic: every kernel variant
the dispatcher can pick (hand-scheduled two- and three-slot, streaming, register-staged) against the oracle."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from tests.gpu_util import dev, host, close_bf16

pytestmark = pytest.mark.gpu


def _shapes(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = int(rng.choice([1, 17, 64, 100, 128, 129, 255, 256, 257, 300, 511, 600, 777]))
        n = int(rng.choice([4, 32, 100, 256, 260, 512, 700, 1028]))
        k = int(rng.choice([32, 96, 128, 256, 384, 512, 768, 1024, 2048]))
        out.append((m, n, k))
    return out


@pytest.mark.parametrize("m,n,k", _shapes(1, 36))
def test_dense_sweep(m, n, k):
    from catccos_amd import ops
    rng = np.random.default_rng(m * 131 + n * 17 + k)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)), "E4M3")
    bq, bsc = O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32)), "E4M3")
    c = ops.mx_gemm(dev(aq), dev(asc), dev(bq), dev(bsc), k)
    bad, worst = close_bf16(host(c), O.mx_gemm_f32(aq, asc, bq, bsc))
    assert bad == 0, (bad, worst)


def _groupings(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        g = int(rng.integers(1, 9))
        scale = int(rng.choice([8, 70, 140, 300, 520]))
        counts = [int(c) for c in rng.integers(0, scale + 1, size=g)]
        if sum(counts) == 0:
            counts[0] = 3
        n = int(rng.choice([64, 256, 320, 768]))
        k = int(rng.choice([128, 256, 512, 1024]))
        out.append((tuple(counts), n, k))
    return out


@pytest.mark.parametrize("counts,n,k", _groupings(2, 24))
def test_grouped_sweep(counts, n, k):
    from catccos_amd import ops
    rng = np.random.default_rng(sum(counts) * 7 + n + k)
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    ws_ = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32)), "E4M3", "lut") for _ in counts]
    wq, ws = np.stack([q for q, _ in ws_]), np.stack([s for _, s in ws_])
    cnt = dev(np.array(counts, dtype=np.int32))
    c = ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k)
    bad, worst = close_bf16(host(c), O.mx_gmm_f32(aq, asc, wq, ws, list(counts)))
    assert bad == 0, (bad, worst)
    if n % 64 == 0:
        # fused SwiGLU + requant on the same operands: dequantised activation within the bound of two chained
        # bf16 roundings and one E4M3 quantisation step
        codes, scales, _ = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k)
        _, _, gq, gs = O.gmm1_swiglu_quant(aq, asc, wq, ws, list(counts))
        deq, deq_g = O.mx_dequant(host(codes), host(scales)), O.mx_dequant(gq, gs)
        bound = 0.13 * np.abs(deq_g) + 2.0 ** -5 * np.abs(deq_g).max(axis=1, keepdims=True) + 1e-6
        assert np.all(np.abs(deq - deq_g) <= bound)


@pytest.mark.parametrize("fmt", ["E4M3", "E2M1"])
@pytest.mark.parametrize("out", ["bf16", "fp16"])
def test_output_pitch_and_edges_are_left_alone(fmt, out):
    """The persistent kernels store their 16-bit output in whole lines through the LDS.  With an output pitch wider than
    n, a ragged last row tile and a ragged last column tile, every element inside equals the tight-pitch call bit for bit
    and every element outside keeps its poison."""
    from catccos_amd import _lib, ops
    m, n, k, ldc, pad_rows = 300, 520, 1024, 536, 3
    rng = np.random.default_rng(77)
    if fmt == "E2M1":
        aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
        bq, bsc = O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1")
        aq, bq = O.pack_fp4(aq), O.pack_fp4(bq)
    else:
        aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)), "E4M3")
        bq, bsc = O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32)), "E4M3")
    a, a_s, b, b_s = dev(aq), dev(asc), dev(bq), dev(bsc)
    tight = ops.mx_gemm(a, a_s, b, b_s, k, fmt, out)
    wide = torch.full((m + pad_rows, ldc), 0x7FC1, dtype=torch.int16, device="cuda")
    lib = _lib.load()
    _lib.check(lib.cmx_mx_gemm(a.data_ptr(), a.stride(0), a_s.data_ptr(), a_s.stride(0), b.data_ptr(), b.stride(0), b_s.data_ptr(),
                               b_s.stride(0), wide.data_ptr(), ldc, m, n, k, ops.FMT[fmt], ops.OUT[out],
                               torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(wide[:m, :n], tight.view(torch.int16))
    assert bool((wide[:m, n:] == 0x7FC1).all()) and bool((wide[m:] == 0x7FC1).all())


@pytest.mark.parametrize("fmt", ["E4M3", "E2M1"])
def test_grouped_output_pitch_and_edges_are_left_alone(fmt):
    """The same for the grouped matmul (ragged groups, one empty, rows past the groups): inside bit-equal to the
    tight-pitch call, outside untouched."""
    from catccos_amd import ops
    counts, n, k, ldc, spare = [700, 0, 900, 650], 520, 1024, 536, 5
    m = sum(counts)
    rng = np.random.default_rng(78)
    if fmt == "E2M1":
        aq, asc = O.mx_quant(rng.uniform(-2, 2, (m + spare, k)).astype(np.float32), "E2M1")
        ws_ = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in counts]
        aq = O.pack_fp4(aq)
        wq = np.stack([O.pack_fp4(q) for q, _ in ws_])
    else:
        aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m + spare, k)).astype(np.float32)), "E4M3")
        ws_ = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32)), "E4M3", "lut") for _ in counts]
        wq = np.stack([q for q, _ in ws_])
    wsc = np.stack([s for _, s in ws_])
    a, a_s, w, w_s = dev(aq), dev(asc), dev(wq), dev(wsc)
    cnt = torch.tensor(counts, dtype=torch.int32, device="cuda")
    tight = ops.mx_gmm(a, a_s, w, w_s, cnt, k, fmt)
    wide = torch.full((m + spare, ldc), 0x7FC1, dtype=torch.int16, device="cuda")
    ops.mx_gmm(a, a_s, w, w_s, cnt, k, fmt, c=wide.view(torch.bfloat16)[:, :n])
    torch.cuda.synchronize()
    assert torch.equal(wide[:m, :n], tight.view(torch.int16)[:m])
    assert bool((wide[:, n:] == 0x7FC1).all()) and bool((wide[m:] == 0x7FC1).all())
