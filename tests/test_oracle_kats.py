"""Literal known-answer tests of the oracle's host-side contracts: every expected number below was worked out by
hand from the reference's text (file:line in each test), none comes from running the function under test."""
import numpy as np

from oracle import mx_oracle as O


# ---- workspace sizing: ascend950_dispatch_ffn_combine_host.h:145-164 ----------------------------------------------
def test_ffn_workspace_bytes_default_run_shape():
    # (m, k, n, E, topK) = (4, 7168, 4096, 16, 6), one rank: rows = 24, meta = 64.  The ten 512-rounded terms:
    terms = [6144,        # R512(R256(4) * 6 * 4)
             344064,      # R512(24 * 7168 * 2)
             512,         # R512(64)
             172032,      # R512(24 * 7168)
             5632,        # R512(24 * R2(224) = 5376)
             98304,       # SwigluRegionBytes(24 * 2048 * 2, 16) = R512(max(98304, 1024))
             49152,       # R512(24 * 2048)
             1536,        # R512(24 * R2(64))
             344064,      # DispatchRegionBytes(344064, 1, 16) = R512(max(344064, 64 + 1024))
             512]         # R512(64)
    assert sum(terms) == 1021952
    assert O.ffn_workspace_bytes(4, 7168, 4096, 1, 1, 16, 6) == 1021952


def test_ffn_workspace_bytes_deepseek_shape():
    # (8192, 7168, 4096, 256, 8): rows = 65536, meta = 1024
    terms = [262144, 939524096, 1024, 469762048, 14680064, 268435456, 134217728, 4194304, 939524096, 1024]
    assert sum(terms) == 2770601984
    assert O.ffn_workspace_bytes(8192, 7168, 4096, 1, 1, 256, 8) == 2770601984


def test_ffn_workspace_bytes_odd_scale_columns_and_ragged_rounding():
    # (150, 96, 192, 4, 2): rows = 300; K/32 = 3 -> R2 = 4 and (N/2)/32 = 3 -> 4: dropping either R2 changes a term
    # (300 * 3 = 900 -> 1024 instead of 300 * 4 = 1200 -> 1536)
    terms = [2048, 57856, 512, 29184, 1536, 57856, 29184, 1536, 57856, 512]
    assert sum(terms) == 238080
    assert O.ffn_workspace_bytes(150, 96, 192, 1, 1, 4, 2) == 238080


def test_ffn_workspace_bytes_two_ranks():
    # (4, 256, 512), rankSize = epSize = 2, 8 experts, topK 2: epr = 4, rows = 16, meta = 2 * 2 * 4 * 4 = 64
    terms = [2048, 8192, 512, 4096, 512, 8192, 4096, 512, 8192, 512]
    assert sum(terms) == 36864
    assert O.ffn_workspace_bytes(4, 256, 512, 2, 2, 8, 2) == 36864


# ---- element acceptance: verify_result.py:188-241, utils.py:97-105 --------------------------------------------------
def _bits(v):
    b = O.f32_to_bf16_bits(np.asarray(v, dtype=np.float32))
    assert np.array_equal(O.bf16_bits_to_f32(b), np.asarray(v, dtype=np.float32)), "test values must be exact in bf16"
    return b


def test_get_rtol_switches_at_2048():
    assert O.get_rtol_bf16(2047) == 2.0 ** -7 and O.get_rtol_bf16(2048) == 2.0 ** -6
    assert O.get_rtol_bf16(1) == 2.0 ** -7 and O.get_rtol_bf16(7168) == 2.0 ** -6


def test_verify_bf16_element_exactly_at_the_tolerance_passes_one_ulp_beyond_fails():
    # |gold| > 1: tolerance = rtol * |gold|.  gold 4, K >= 2048 -> 4 * 2^-6 = 0.0625; bf16 spacing in [4, 8) is 2^-5
    gold = np.array([4.0] + [1.0] * 7, dtype=np.float32)          # seven exact elements keep the mean bias small
    ok, err, eb = O.verify_bf16(_bits([4.0625] + [1.0] * 7), gold, 2048)
    assert ok and err == 0 and eb == 2.0 ** -6 / 8
    ok, err, _ = O.verify_bf16(_bits([4.09375] + [1.0] * 7), gold, 2048)
    assert not ok and err == 1
    # the same element under K < 2048 (rtol 2^-7 -> 0.03125) already fails at 4.0625
    ok, err, _ = O.verify_bf16(_bits([4.0625] + [1.0] * 7), gold, 2047)
    assert not ok and err == 1
    # |gold| < 1: the tolerance is absolute (max(1, |gold|) = 1).  gold 0.5, K 2047: 0.5 + 2^-7 passes, one ulp
    # (2^-8) more fails -- and passes again with the K >= 2048 tolerance
    gold = np.array([0.5] + [0.25] * 7, dtype=np.float32)
    assert O.verify_bf16(_bits([0.5 + 2.0 ** -7] + [0.25] * 7), gold, 2047)[0]
    assert not O.verify_bf16(_bits([0.5 + 2.0 ** -7 + 2.0 ** -8] + [0.25] * 7), gold, 2047)[0]
    assert O.verify_bf16(_bits([0.5 + 2.0 ** -7 + 2.0 ** -8] + [0.25] * 7), gold, 2048)[0]
    # negative side of the tolerance
    assert O.verify_bf16(_bits([-4.0625] + [1.0] * 7), -np.array([4.0] + [-1.0] * 7, dtype=np.float32), 2048)[0]


def test_verify_bf16_mean_bias_rule():
    # every element inside its own tolerance (2^-6) but all off to the same side by 2^-7: eb = 2^-7 passes ...
    gold = np.zeros(64, dtype=np.float32)
    ok, err, eb = O.verify_bf16(_bits(np.full(64, 2.0 ** -7)), gold, 4096)
    assert ok and err == 0 and eb == 2.0 ** -7
    # ... and by 2^-7 (1 + 2^-7) fails on the bias alone
    ok, err, eb = O.verify_bf16(_bits(np.full(64, 2.0 ** -7 * (1 + 2.0 ** -7))), gold, 4096)
    assert not ok and err == 0 and eb > 2.0 ** -7
    # opposite signs cancel
    v = np.full(64, 2.0 ** -7 * (1 + 2.0 ** -7), dtype=np.float32)
    v[::2] *= -1
    assert O.verify_bf16(_bits(v), gold, 4096)[0]


def test_verify_bf16_non_finite_positions_must_coincide():
    gold = np.array([1.0, np.inf, 2.0, np.nan], dtype=np.float32)
    same = np.array([0x3F80, 0x7F80, 0x4000, 0x7FC0], dtype=np.uint16)          # 1, Inf, 2, NaN
    assert O.verify_bf16(same, gold, 64)[0]                                     # both replaced by zero, then equal
    moved = np.array([0x7F80, 0x3F80, 0x4000, 0x7FC0], dtype=np.uint16)         # Inf in another place
    ok, err, eb = O.verify_bf16(moved, gold, 64)
    assert not ok and err == -1
    # an Inf where the golden is finite is a mismatch even if everything else is exact
    assert not O.verify_bf16(np.array([0x3F80, 0x7F80, 0x7F80, 0x7FC0], dtype=np.uint16), gold, 64)[0]
    # -Inf against +Inf counts as the same position (the rule looks at finiteness only)
    assert O.verify_bf16(np.array([0x3F80, 0xFF80, 0x4000, 0x7FC0], dtype=np.uint16), gold, 64)[0]


# ---- double-golden acceptance: verify_result.py:117-134, 244-306 ----------------------------------------------------
def test_double_golden_rule_thresholds():
    gold = np.ones(64, dtype=np.float32)
    low = _bits(np.ones(64))                                    # the bf16 golden is exact here: denominators are 2^-8
    out = np.ones(64, dtype=np.float32)
    out[0] = 1 + 2.0 ** -7                                      # one bf16 ulp off
    ok, r_max, r_mean, r_rmse, eb = O.verify_double_golden_bf16(_bits(out), gold, low)
    assert ok
    assert abs(r_max - 2.0) < 1e-5                              # 2^-7 / (1 + 1e-7) / 2^-8
    assert abs(r_mean - 2.0 / 64) < 1e-6
    assert abs(r_rmse - 2.0 / 8) < 1e-6                         # sqrt(2^-14 / 64) / 2^-8
    assert eb == 2.0 ** -7 / 64
    # one element 12 * 2^-8 off (six ulps): only the maximum-error rule (< 10) trips -- mean ratio 12/64, rmse ratio
    # 12/8, bias 12 * 2^-8 / 64
    out[0] = 1 + 12 * 2.0 ** -8
    ok, r_max, r_mean, r_rmse, eb = O.verify_double_golden_bf16(_bits(out), gold, low)
    assert not ok and 11.99 < r_max < 12.01 and abs(r_mean - 12 / 64) < 1e-5 and abs(r_rmse - 1.5) < 1e-5 and eb <= 2.0 ** -7
    # 10 * 2^-8 off: the relative error divides by |gold| + 1e-7, so the ratio stays a hair below 10 and passes
    out[0] = 1 + 10 * 2.0 ** -8
    ok, r_max, *_ = O.verify_double_golden_bf16(_bits(out), gold, low)
    assert ok and 9.99 < r_max < 10.0
    # the low golden's own error relaxes the bound: with the bf16 golden two ulps off at the same place, the output
    # that failed above passes (12 * 2^-8 against 2^-6: ratio 3)
    low2 = _bits(np.where(np.arange(64) == 0, 1 + 2.0 ** -6, 1.0))
    out[0] = 1 + 12 * 2.0 ** -8
    ok, r_max, *_ = O.verify_double_golden_bf16(_bits(out), gold, low2)
    assert ok and abs(r_max - 3.0) < 1e-5


def test_double_golden_mean_and_rmse_rules():
    gold = np.ones(64, dtype=np.float32)
    low = _bits(np.ones(64))
    # every element 2 * 2^-8 off (one ulp): max ratio 2 passes, the RMSE ratio is exactly 2 and fails (< 2 is
    # required; the mean ratio divides by |gold| + 1e-7 and stays a hair below 2)
    ok, r_max, r_mean, r_rmse, _ = O.verify_double_golden_bf16(_bits(np.full(64, 1 + 2.0 ** -7)), gold, low)
    assert not ok and r_max < 10 and 1.9999 < r_mean < 2.0 and r_rmse == 2.0
    # alternate signs: same figures (they use absolute errors), the bias is zero
    v = np.where(np.arange(64) % 2 == 0, 1 + 2.0 ** -7, 1 - 2.0 ** -7)
    ok, _, r_mean, _, eb = O.verify_double_golden_bf16(_bits(v), gold, low)
    assert not ok and eb == 0.0 and abs(r_mean - 2.0) < 1e-5
    # half of the elements off: mean ratio 1, rmse ratio sqrt(1/2) * 2 = 1.414: passes
    v = np.where(np.arange(64) % 2 == 0, 1 + 2.0 ** -7, 1.0)
    assert O.verify_double_golden_bf16(_bits(v), gold, low)[0]
    # non-finite mismatch
    bad = _bits(np.ones(64)).copy()
    bad[3] = 0x7F80
    assert not O.verify_double_golden_bf16(bad, gold, low)[0]
