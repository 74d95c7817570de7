"""Known-answer tests of the block-scaled MFMA register layout the GEMM kernels assume
(v_mfma_scale_f32_32x32x64_f8f6f4): lane l feeds row l%32.  FP4: its 16 bytes are the 32
consecutive K elements of block l/32.  8-bit formats: registers 0-3 hold k = 16*(l/32) + [0,16)
of block 0 and registers 4-7 the same slice of block 1.  Byte `opsel` of the lane's scale
register scales block l/32 of its row.  Accumulator register r of lane l is
(row 8*(r/4) + 4*(l/32) + r%4 of the first operand, row l%32 of the second)."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from tests.gpu_util import dev, host, mfma_raw_probe

pytestmark = pytest.mark.gpu


def _regs_fp8(codes):       # codes u8 [32, 64] -> int32 [64, 8]
    regs = np.zeros((64, 32), dtype=np.uint8)
    for l in range(64):
        h = l // 32
        regs[l, :16] = codes[l % 32, 16 * h:16 * h + 16]
        regs[l, 16:] = codes[l % 32, 32 + 16 * h:32 + 16 * h + 16]
    return regs.view(np.int32).reshape(64, 8)


def _regs_fp4(packed):      # packed u8 [32, 32] (64 nibbles per row) -> int32 [64, 8] (upper 4 unused)
    regs = np.zeros((64, 32), dtype=np.uint8)
    for l in range(64):
        regs[l, :16] = packed[l % 32, 16 * (l // 32):16 * (l // 32) + 16]
    return regs.view(np.int32).reshape(64, 8)


def _scale_regs(scales, opsel):   # scales u8 [32, 2] -> int32 [64] with the lane's byte at position opsel
    rng = np.random.default_rng(99)
    r = rng.integers(0, 256, size=(64, 4), dtype=np.uint8)      # junk in the unselected bytes
    for l in range(64):
        r[l, opsel] = scales[l % 32, l // 32]
    return r.view(np.int32).reshape(64)


def _unpack_acc(out):       # [64, 16] -> [32, 32] (first-operand row, second-operand row)
    c = np.zeros((32, 32), dtype=np.float32)
    for l in range(64):
        for r in range(16):
            c[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32] = out[l, r]
    return c


@pytest.mark.parametrize("opsel", [0, 2, 3])
def test_mfma_32x32x64_fp8_layout(opsel):
    from catccos_amd import ops
    rng = np.random.default_rng(opsel)
    w, ws = O.mx_quant(rng.standard_normal((32, 64)).astype(np.float32) * 3)
    a, as_ = O.mx_quant(rng.standard_normal((32, 64)).astype(np.float32) * 0.2)
    ws, as_ = ws[:, :2], as_[:, :2]
    ws[5, 1] += 3; as_[7, 0] -= 2          # make the two K blocks of a row scale differently
    out = mfma_raw_probe(dev(_regs_fp8(w)), dev(_regs_fp8(a)), dev(_scale_regs(ws, opsel)),
                             dev(_scale_regs(as_, opsel)), "E4M3", opsel, 0)
    got = _unpack_acc(host(out))
    want = O.mx_dequant(w, ws).astype(np.float64) @ O.mx_dequant(a, as_).astype(np.float64).T
    # 8-bit products are aligned to the largest one inside the MFMA, which drops ~2^-13 of it;
    # a wrong lane/byte/scale mapping is off by O(1), not O(1e-3)
    assert np.allclose(got, want, rtol=1e-3, atol=5e-3), np.abs(got - want).max()


def test_mfma_32x32x64_fp4_layout():
    from catccos_amd import ops
    rng = np.random.default_rng(7)
    w, ws = O.mx_quant(rng.uniform(-2, 2, (32, 64)).astype(np.float32), "E2M1")
    a, as_ = O.mx_quant(rng.uniform(-2, 2, (32, 64)).astype(np.float32), "E2M1")
    out = mfma_raw_probe(dev(_regs_fp4(O.pack_fp4(w))), dev(_regs_fp4(O.pack_fp4(a))), dev(_scale_regs(ws[:, :2], 1)),
                             dev(_scale_regs(as_[:, :2], 1)), "E2M1", 1, 0)
    got = _unpack_acc(host(out))
    want = O.mx_dequant(w, ws, "E2M1").astype(np.float64) @ O.mx_dequant(a, as_, "E2M1").astype(np.float64).T
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5), np.abs(got - want).max()


def test_mfma_one_hot_locates_every_operand_byte():
    """A single 1.0 at (row i, k) times an all-ones second operand lights up row i only, for every k."""
    from catccos_amd import ops
    ones = np.full((32, 64), 0x38, dtype=np.uint8)
    unit = np.full((32, 2), 127, dtype=np.uint8)
    for (i, k) in [(0, 0), (3, 31), (17, 32), (31, 63), (9, 40)]:
        w = np.zeros((32, 64), dtype=np.uint8)
        w[i, k] = 0x40      # 2.0
        out = mfma_raw_probe(dev(_regs_fp8(w)), dev(_regs_fp8(ones)), dev(_scale_regs(unit, 0)),
                                 dev(_scale_regs(unit, 0)), "E4M3", 0, 0)
        got = _unpack_acc(host(out))
        want = np.zeros((32, 32), dtype=np.float32)
        want[i, :] = 2.0
        assert np.array_equal(got, want), (i, k)
