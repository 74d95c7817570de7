"""Pins the numpy oracle's quantizer against known answers, a library cast that
is not reference code (torch CPU float8), brute-force definitions and invariants."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O


def all_bf16_f32(limit=None):
    bits = np.arange(65536, dtype=np.uint16)
    v = O.bf16_bits_to_f32(bits)
    ok = np.isfinite(v)
    if limit is not None:
        ok &= np.abs(v) <= limit
    return v[ok]


# ---- E8M0: known answers fixed by floor(log2 amax) - emax -----------------------------------
@pytest.mark.parametrize("amax,emax,byte", [
    (1.0, 8, 119), (448.0, 8, 127), (511.0, 8, 127), (512.0, 8, 128), (2.0 ** -20, 8, 99), (0.0, 8, 127),
    (1.0, 2, 125), (6.0, 2, 127), (7.9, 2, 127), (8.0, 2, 128), (1e-13, 8, 127), (1.0, 15, 112), (1.0, 0, 127),
])
def test_e8m0_known_answers(amax, emax, byte):
    e = O.e8m0_exp(np.array([amax], dtype=np.float32), emax)
    assert int(O.e8m0_byte(e)[0]) == byte


def test_e8m0_matches_floor_log2_everywhere():
    v = all_bf16_f32()
    v = np.abs(v[np.abs(v) >= 1e-12])
    want = np.clip(np.floor(np.log2(v.astype(np.float64))) - 8, -128, 127).astype(np.int32)
    assert np.array_equal(O.e8m0_exp(v, 8), want)


# ---- bf16 RNE --------------------------------------------------------------------------------
def test_bf16_rne_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 50,
                        np.array([0.0, -0.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.3895e38, 1e-40], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), want)
    assert np.array_equal(O.bf16_bits_to_f32(want), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


# ---- FP8 RNE vs the torch CPU cast (library, not reference code) -----------------------------
def _torch_fp8(x, dt):
    return torch.from_numpy(np.ascontiguousarray(x)).to(dt).view(torch.uint8).numpy()


def test_e4m3_rne_all_bf16_and_random():
    rng = np.random.default_rng(1)
    v = all_bf16_f32(448.0)
    for s in (1.0, 0.75, 1.0 / 3, 2.0 ** -7):
        y = (v * np.float32(s)).astype(np.float32)
        assert np.array_equal(O.e4m3_encode_rne(y), _torch_fp8(y, torch.float8_e4m3fn))
    y = np.clip(rng.standard_normal(500000).astype(np.float32) * 100, -448, 448)
    assert np.array_equal(O.e4m3_encode_rne(y), _torch_fp8(y, torch.float8_e4m3fn))
    # exact midpoints between neighbours: ties go to the even mantissa
    tab = O.e4m3_table()[:127].astype(np.float64)
    mid = ((tab[:-1] + tab[1:]) / 2).astype(np.float32)
    assert np.array_equal(O.e4m3_encode_rne(mid), _torch_fp8(mid, torch.float8_e4m3fn))
    assert np.array_equal(O.e4m3_encode_rne(-mid), _torch_fp8(-mid, torch.float8_e4m3fn))


def test_e4m3_rne_special_cases():
    y = np.array([448.0, -448.0, 0.0, -0.0, 2.0 ** -9, 2.0 ** -10, -(2.0 ** -11), 2.0 ** -6, 464.0 - 16], dtype=np.float32)
    got = O.e4m3_encode_rne(y)
    assert list(got) == [0x7E, 0xFE, 0x00, 0x80, 0x01, 0x00, 0x80, 0x08, 0x7E]


def test_e5m2_rne_all_bf16():
    v = all_bf16_f32(57344.0)
    assert np.array_equal(O.e5m2_encode_rne(v), _torch_fp8(v, torch.float8_e5m2))
    rng = np.random.default_rng(2)
    y = np.clip(rng.standard_normal(300000).astype(np.float32) * 1000, -57344, 57344)
    assert np.array_equal(O.e5m2_encode_rne(y), _torch_fp8(y, torch.float8_e5m2))


def test_decode_tables_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    fin = np.isfinite(t)
    assert np.array_equal(O.e4m3_table()[fin], t[fin])
    assert O.e4m3_table()[127] == 448.0 and O.e4m3_table()[255] == -448.0   # reference table, not NaN
    t5 = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    keep = np.isfinite(t5) & (np.abs(t5) <= 57344)
    assert np.array_equal(O.e5m2_table()[keep], t5[keep])


# ---- LUT mode: vectorised form vs the arg-min definition -------------------------------------
@pytest.mark.parametrize("fmt,lim", [("E4M3", 448.0), ("E5M2", 57344.0)])
def test_fp8_lut_equals_argmin_definition(fmt, lim):
    v = all_bf16_f32(lim)
    tab = O.e4m3_table() if fmt == "E4M3" else O.e5m2_table()
    mid = ((tab[:126].astype(np.float64) + tab[1:127]) / 2).astype(np.float32)
    y = np.concatenate([v, mid, -mid, (v * np.float32(0.3)).astype(np.float32)])
    assert np.array_equal(O.fp8_encode_lut(y, fmt), O.fp8_encode_lut_argmin(y, fmt))


def test_e4m3_lut_properties():
    v = np.sort(all_bf16_f32(448.0))
    c = O.fp8_encode_lut(v, "E4M3")
    d = O.decode(c, "E4M3")
    assert np.all(np.diff(d) >= 0)                               # monotone
    assert not np.any(c == 0x80) and not np.any((c & 0x7F) == 0x7F)   # -0 -> +0, never 0x7F
    pos = v[v > 0]
    assert np.array_equal(O.decode(O.fp8_encode_lut(-pos, "E4M3"), "E4M3"), -O.decode(O.fp8_encode_lut(pos, "E4M3"), "E4M3"))
    grid = O.e4m3_table()[:127]
    assert np.array_equal(O.fp8_encode_lut(grid, "E4M3"), np.arange(127, dtype=np.uint8))   # idempotent
    # ties go to the smaller magnitude; RNE and LUT differ only on exact midpoints and on -0
    mid = ((grid[:-1].astype(np.float64) + grid[1:]) / 2).astype(np.float32)
    assert np.array_equal(O.fp8_encode_lut(mid, "E4M3"), np.arange(126, dtype=np.uint8))
    r = O.e4m3_encode_rne(v)
    differ = r != c
    is_mid = np.isin(np.abs(v), mid)
    assert np.all(is_mid[differ] | (r[differ] == 0x80))


# ---- FP4 ------------------------------------------------------------------------------------
def test_fp4_tables():
    assert list(O.fp4_table("E2M1")[:8]) == [0, 0.5, 1, 1.5, 2, 3, 4, 6]
    assert list(O.fp4_table("E1M2")[:8]) == [0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75]
    assert np.array_equal(O.fp4_table("E2M1")[8:], -O.fp4_table("E2M1")[:8])


def test_fp4_lut_ties_and_bruteforce():
    y = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.0, -5.0, 6.0, 0.26, 5.01], dtype=np.float32)
    assert list(O.fp4_encode_lut(y)) == [0, 1, 2, 3, 4, 5, 6, 0, 0, 14, 7, 1, 7]
    v = all_bf16_f32(6.0)
    tab = O.fp4_table("E2M1")
    want = np.argmin(np.abs(v[:, None] - tab[None, :]), axis=1).astype(np.uint8)   # first index wins
    assert np.array_equal(O.fp4_encode_lut(v), want)


def test_fp4_rne_ties_to_even():
    y = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.75, 0.2, 5.5, -6.0], dtype=np.float32)
    assert list(O.fp4_encode_rne(y)) == [0, 2, 2, 4, 4, 6, 6, 8, 10, 0, 7, 15]
    v = all_bf16_f32(6.0)
    c = O.fp4_encode_rne(v)
    err = np.abs(O.decode(c, "E2M1") - v)
    tab = O.fp4_table("E2M1")
    best = np.min(np.abs(v[:, None] - tab[None, :]), axis=1)
    assert np.array_equal(err, best)                              # always a nearest value


def test_e1m2_lut_and_rne_against_the_grid_k_over_4():
    """E1M2 values are k/4, k = 0..7 (gen_mx_quant_allgather_data.py:65-72, 352-376): the table encode is the
    first arg-min over the 16 entries, RNE is round-half-even of 4|y| -- both checked by brute force over every
    bf16 value up to the clip, plus the ties written out."""
    y = np.array([0.125, 0.375, 0.625, 0.875, 1.125, 1.375, 1.625, -0.125, -0.0, -1.7, 1.75, 0.13], dtype=np.float32)
    assert list(O.fp4_encode_lut(y, "E1M2")) == [0, 1, 2, 3, 4, 5, 6, 0, 0, 15, 7, 1]
    assert list(O.fp4_encode_rne(y, "E1M2")) == [0, 2, 2, 4, 4, 6, 6, 8, 8, 15, 7, 1]
    v = all_bf16_f32(1.75)
    tab = O.fp4_table("E1M2")
    want = np.argmin(np.abs(v[:, None] - tab[None, :]), axis=1).astype(np.uint8)
    assert np.array_equal(O.fp4_encode_lut(v, "E1M2"), want)
    k = np.rint(np.abs(v).astype(np.float64) * 4).astype(np.int64)        # numpy rint: half to even
    assert np.array_equal(O.fp4_encode_rne(v, "E1M2"), (k | np.where(np.signbit(v), 8, 0)).astype(np.uint8))
    # block exponent: emax 0, so amax in [1, 2) keeps scale 2^0 and amax 1.9 clips to 1.75
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :4] = [1.9, -0.3, 0.375, 1.0]
    q, s = O.mx_quant(x, "E1M2", "lut")
    assert s[0, 0] == 127 and q[0, :4].tolist() == [7, 9, 1, 4]
    x[0, 0] = 4.0                                                          # floor(log2 4) - 0 = 2
    q, s = O.mx_quant(x, "E1M2", "lut")
    assert s[0, 0] == 129 and q[0, :4].tolist() == [4, 0, 0, 1]          # 1.0, -0.075 -> +0, 0.094 -> 0, 0.25


def test_fp4_pack_closed_form():
    rng = np.random.default_rng(3)
    c = rng.integers(0, 16, size=(5, 64), dtype=np.uint8)
    p = O.pack_fp4(c)
    assert np.array_equal(p, c[:, 0::2] + 16 * c[:, 1::2])
    assert np.array_equal(O.unpack_fp4(p), c)
    assert O.pack_fp4(np.array([[1, 2, 3]], dtype=np.uint8)).tolist() == [[0x21, 0x03]]


# ---- block quantizer -------------------------------------------------------------------------
def test_mx_quant_block_known_answers():
    x = np.zeros((2, 96), dtype=np.float32)
    x[0, 0:32] = 511.0            # scale 2^0, elements clip to 448
    x[0, 32:64] = 1.0             # amax 1 -> byte 119, 1/2^-8 = 256 -> code of 256
    x[1, 0] = -3.0                # floor(log2 3)=1 -> e=-7; -3*128=-384 -> 0xFC
    q, s = O.mx_quant(x, "E4M3", "rne")
    assert s.shape == (2, 4)      # 3 blocks padded to an even count with 1.0
    assert s[0].tolist() == [127, 119, 127, 127] and s[1].tolist() == [120, 127, 127, 127]
    assert np.all(q[0, 0:32] == 0x7E) and np.all(q[0, 32:64] == 0x78) and q[1, 0] == 0xFC
    assert np.all(q[0, 64:] == 0) and np.all(q[1, 1:] == 0)


@pytest.mark.parametrize("fmt,mode", [("E4M3", "rne"), ("E4M3", "lut"), ("E5M2", "rne"), ("E2M1", "lut"), ("E2M1", "rne"),
                                      ("E1M2", "lut"), ("E1M2", "rne")])
def test_mx_quant_is_idempotent_on_its_own_output(fmt, mode):
    """The reference's byte-exact protocol feeds the quantizer its own dequantized
    output re-encoded as bf16 (ascend950_mx_quant_allgather/scripts/run.sh:78-141)."""
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((64, 256)) * 10 - 5).astype(np.float32)
    q, s = O.mx_quant(x, fmt, mode)
    deq = O.mx_dequant(q, s, fmt)
    xb = O.f32_to_bf16_bits(deq)
    assert np.array_equal(O.bf16_bits_to_f32(xb), deq)            # exactly representable in bf16
    q2, s2 = O.mx_quant_bf16(xb, fmt, mode)
    assert np.array_equal(q2, q) and np.array_equal(s2, s)


def test_mx_quant_rne_matches_torch_pipeline():
    """Independent pipeline: torch amax / exp2 / division / clamp / float8 cast."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((128, 512)).astype(np.float32)
    x[rng.random(x.shape) < 0.001] *= 100
    x = O.bf16_round(x)
    q, s = O.mx_quant(x, "E4M3", "rne")
    t = torch.from_numpy(x).view(128, 16, 32)
    amax = t.abs().amax(-1)
    e = torch.floor(torch.log2(amax.double())).to(torch.int32) - 8
    scale = torch.exp2(e.float())
    want = (t / scale[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).reshape(128, 512).numpy()
    assert np.array_equal(q, want)
    assert np.array_equal(s, (e + 127).to(torch.uint8).numpy())
    ws = torch.exp2(e.float()).to(torch.float8_e8m0fnu).view(torch.uint8).numpy()
    assert np.array_equal(s, ws)


def test_mx_dequant_matches_torch():
    rng = np.random.default_rng(6)
    q = rng.integers(0, 256, size=(16, 128), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0
    s = rng.integers(100, 140, size=(16, 4), dtype=np.uint8)
    want = torch.from_numpy(q).view(torch.float8_e4m3fn).float() * torch.from_numpy(s).view(torch.float8_e8m0fnu).float().repeat_interleave(32, dim=1)
    assert np.array_equal(O.mx_dequant(q, s, "E4M3"), want.numpy())


def test_ragged_columns_pad_with_zero_and_unit_scale():
    x = np.ones((1, 40), dtype=np.float32)
    q, s = O.mx_quant(x, "E4M3", "rne")
    assert q.shape == (1, 40) and s.shape == (1, 2) and s.tolist() == [[119, 119]]
    x = np.ones((1, 20), dtype=np.float32)
    q, s = O.mx_quant(x, "E4M3", "rne")
    assert s.tolist() == [[119, 127]]
