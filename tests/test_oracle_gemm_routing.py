"""Pins the oracle's GEMM, SwiGLU, routing, combine and sizing restatements."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W


def _rand_mx(rng, m, k, fmt="E4M3"):
    x = rng.standard_normal((m, k)).astype(np.float32)
    return O.mx_quant(x, fmt)


def test_gemm_all_unit_scales_is_plain_fp8_gemm():
    rng = np.random.default_rng(0)
    a = rng.integers(0, 0x60, size=(8, 64), dtype=np.uint8) | (rng.integers(0, 2, size=(8, 64), dtype=np.uint8) << 7)
    b = rng.integers(0, 0x60, size=(12, 64), dtype=np.uint8) | (rng.integers(0, 2, size=(12, 64), dtype=np.uint8) << 7)
    sa = np.full((8, 2), 127, dtype=np.uint8)
    sb = np.full((12, 2), 127, dtype=np.uint8)
    ta = torch.from_numpy(a).view(torch.float8_e4m3fn).double()
    tb = torch.from_numpy(b).view(torch.float8_e4m3fn).double()
    want = (ta @ tb.T).numpy()
    got = O.mx_gemm_f32(a, sa, b, sb)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-3)   # fp32 accumulation of O(1e3) terms


def test_gemm_one_hot_rows_copy_dequantized_weight_rows():
    rng = np.random.default_rng(1)
    bq, bs = _rand_mx(rng, 16, 128)
    a = np.zeros((4, 128), dtype=np.uint8)
    a[0, 5] = 0x38          # 1.0
    a[1, 40] = 0xB8         # -1.0
    a[2, 127] = 0x40        # 2.0
    sa = np.full((4, 4), 127, dtype=np.uint8)
    sa[2, 3] = 129          # block 3 scaled by 4 -> 8 * column 127
    got = O.mx_gemm_f32(a, sa, bq, bs)
    deq_b = O.mx_dequant(bq, bs)
    assert np.array_equal(got[0], deq_b[:, 5]) and np.array_equal(got[1], -deq_b[:, 40])
    assert np.array_equal(got[2], 8 * deq_b[:, 127]) and np.all(got[3] == 0)


def test_gemm_block_scale_formula_in_float64():
    """C[m,n] = sum_kb 2^(sa+sb-254) * sum_{k in kb} a*b  evaluated in float64."""
    rng = np.random.default_rng(2)
    aq, asc = _rand_mx(rng, 6, 96)
    bq, bsc = _rand_mx(rng, 5, 96)
    av, bv = O.decode(aq, "E4M3").astype(np.float64), O.decode(bq, "E4M3").astype(np.float64)
    want = np.zeros((6, 5))
    for kb in range(3):
        part = av[:, kb * 32:(kb + 1) * 32] @ bv[:, kb * 32:(kb + 1) * 32].T
        sc = 2.0 ** (asc[:, kb].astype(np.float64)[:, None] + bsc[:, kb].astype(np.float64)[None, :] - 254)
        want += part * sc
    assert np.allclose(O.mx_gemm_f32(aq, asc, bq, bsc), want, rtol=1e-5, atol=1e-6)


def test_fp4_gemm_against_float64():
    rng = np.random.default_rng(3)
    aq, asc = O.mx_quant(rng.uniform(-2, 2, (8, 64)).astype(np.float32), "E2M1")
    bq, bsc = O.mx_quant(rng.uniform(-2, 2, (8, 64)).astype(np.float32), "E2M1")
    want = O.mx_dequant(aq, asc, "E2M1").astype(np.float64) @ O.mx_dequant(bq, bsc, "E2M1").astype(np.float64).T
    assert np.allclose(O.mx_gemm_f32(aq, asc, bq, bsc, "E2M1", "E2M1"), want, rtol=1e-6)


def test_grouped_gemm_equals_per_group_gemm_and_handles_empty_groups():
    rng = np.random.default_rng(4)
    counts = np.array([3, 0, 5, 0, 2], dtype=np.int32)
    aq, asc = _rand_mx(rng, 10, 64)
    w = [_rand_mx(rng, 8, 64) for _ in counts]
    wq, ws = np.stack([x[0] for x in w]), np.stack([x[1] for x in w])
    got = O.mx_gmm_f32(aq, asc, wq, ws, counts)
    off = O.group_offsets(counts)
    assert off.tolist() == [0, 3, 3, 8, 8, 10]
    for g in range(5):
        lo, hi = off[g], off[g + 1]
        assert np.array_equal(got[lo:hi], O.mx_gemm_f32(aq[lo:hi], asc[lo:hi], wq[g], ws[g]))


def test_swiglu_matches_torch_float32():
    rng = np.random.default_rng(5)
    h = O.f32_to_bf16_bits(rng.standard_normal((32, 128)).astype(np.float32) * 4)
    t = torch.from_numpy(O.bf16_bits_to_f32(h))
    act, gate = t.chunk(2, dim=-1)
    want = (act * torch.sigmoid(act) * gate).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.swiglu_bf16(h)
    # exp/sigmoid differ by at most an fp32 ulp between libraries: allow the bf16 result to
    # differ by one bf16 ulp on a tiny fraction of elements, never more.
    d = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert d.max() <= 1 and np.mean(d != 0) < 2e-3
    z = np.zeros((1, 4), dtype=np.uint16)
    assert np.all(O.swiglu_bf16(z) == 0)


# ---- routing -----------------------------------------------------------------------------------
def test_routing_is_a_stable_sort():
    rng = np.random.default_rng(6)
    idx = rng.integers(0, 7, size=(50, 4)).astype(np.int32)
    s2s, inv, counts = O.moe_init_routing(idx, 9)
    flat = idx.reshape(-1)
    assert sorted(s2s.tolist()) == list(range(200))
    keys = flat[s2s]
    assert np.all(np.diff(keys) >= 0)
    same = np.diff(keys) == 0
    assert np.all(np.diff(s2s)[same] > 0)                          # source order kept within a key
    assert np.array_equal(inv[s2s], np.arange(200)) and np.array_equal(s2s[inv], np.arange(200))
    assert counts.tolist() == np.bincount(flat, minlength=9).tolist() and counts.dtype == np.int32
    want = torch.argsort(torch.from_numpy(flat.astype(np.int64)), stable=True).numpy()
    assert np.array_equal(s2s, want)


def test_balanced_routing_counts():
    """examples/utils/test_moe_routing.py:8-33"""
    routes = O.balanced_expert_idx(512, 16, 6, 4)
    assert np.bincount(routes.reshape(-1), minlength=16).tolist() == [768] * 16
    assert all(len(set(r)) == 6 for r in routes.reshape(-1, 6).tolist())
    c = np.bincount(O.balanced_expert_idx(7, 5, 3, 2).reshape(-1), minlength=5)
    assert c.max() - c.min() <= 1
    with pytest.raises(ValueError):
        O.balanced_expert_idx(8, 4, 5, 1)


def test_scheduler_prefix_known_answers():
    """tests/comm_block_scheduler_alltoallv_gmm/test_comm_block_scheduler_alltoallv_gmm.cpp:46-100:
    tokens i+1, rank 2, EP 4, 2 experts per rank -> prevSum 42 (core 1), 0 (core 4), 10 (core 0)."""
    tok = np.arange(1, 33, dtype=np.int32)
    assert O.src_prev_sum(tok, 1, 2, 4, 2) == 42
    assert O.src_prev_sum(tok, 4, 2, 4, 2) == 0
    assert O.src_prev_sum(tok, 0, 2, 4, 2) == 10
    cs = O.cumsum_for_mm(tok, 2, 4, 2)
    assert cs.tolist() == [[5, 6], [18, 20], [39, 42], [68, 72]]
    assert O.cumsum_for_mm(np.array([3, 0, 4]), 0, 1, 3).tolist() == [[3, 0, 4]]   # EP=1: identity


# ---- combine -----------------------------------------------------------------------------------
def test_combine_bruteforce_and_order():
    rng = np.random.default_rng(7)
    t, k, h = 6, 3, 8
    idx = np.stack([rng.permutation(5)[:k] for _ in range(t)]).astype(np.int32)
    s2s, inv, counts = O.moe_init_routing(idx, 5)
    y = O.f32_to_bf16_bits(rng.standard_normal((t * k, h)).astype(np.float32))
    p = rng.random((t, k)).astype(np.float32)
    got = O.unpermute_combine(y, inv, p)
    yf = O.bf16_bits_to_f32(y)
    for tok in range(t):
        acc = None
        for kk in range(k):
            term = np.float32(p[tok, kk]) * yf[inv[tok * k + kk]]
            acc = term if acc is None else (acc + term).astype(np.float32)
        assert np.array_equal(got[tok], O.f32_to_bf16_bits(acc))
    # weights one-hot -> a pure gather
    p1 = np.zeros((t, k), dtype=np.float32); p1[:, 1] = 1
    assert np.array_equal(O.unpermute_combine(y, inv, p1), y[inv.reshape(t, k)[:, 1]])
    # index beyond the permuted rows contributes nothing
    inv2 = inv.copy(); inv2[0] = t * k + 5
    g2 = O.unpermute_combine(y, inv2, p)
    acc = (np.float32(p[0, 1]) * yf[inv[1]] + np.float32(0)).astype(np.float32)
    acc = (acc + np.float32(p[0, 2]) * yf[inv[2]]).astype(np.float32)
    assert np.array_equal(g2[0], O.f32_to_bf16_bits(acc))


def test_packed_row_layout():
    assert O.packed_row_bytes(7168) == 7392 and O.packed_row_bytes(256) == 288
    rng = np.random.default_rng(8)
    x = O.f32_to_bf16_bits(rng.standard_normal((4, 64)).astype(np.float32))
    idx = np.array([[1, 0], [0, 2], [2, 1], [0, 1]], dtype=np.int32)
    s2s, inv, counts = O.moe_init_routing(idx, 3)
    packed = O.quant_scatter_packed(x, inv, 2)
    q, s = O.mx_quant_bf16(x)
    assert packed.shape == (8, 96)
    for i in range(8):
        tok = s2s[i] // 2
        assert np.array_equal(packed[i, :64], q[tok]) and np.array_equal(packed[i, 64:66], s[tok])
        assert np.all(packed[i, 66:] == 0)


# ---- sizing ------------------------------------------------------------------------------------
def test_moe_ready_and_ub_known_answers():
    """tests/ascend950/test_moe_ready_capacity.cpp:18-19, test_moe_ub_capacity.cpp:19-38"""
    assert O.moe_ready_swiglu_region_bytes(1024, 32) == 2048
    assert O.moe_ready_dispatch_region_bytes(1024, 2, 32) == 2560
    assert O.moe_ub_unpermute_bytes(512, 2048, 8, 48) == 37760
    assert O.moe_ub_input_quant_bytes(2048) == 12928 and O.moe_ub_dispatch_bytes(2048) == 8448
    assert O.moe_ub_unpermute_bytes(1, 256, 1, 48) == 9536
    assert O.moe_ub_fits(1, 14336, 8, 48) and not O.moe_ub_fits(1, 14592, 8, 48) and not O.moe_ub_fits(1, 2048, 8, 0)
    assert O.moe_ub_fits(28800, 2048, 46, 48) and not O.moe_ub_fits(28800, 2048, 47, 48)
    assert O.moe_ub_fits(1, 7168, 6, 48) and O.moe_ub_fits(512, 2048, 8, 48)
    for ranks in (2, 4, 8):
        for experts in (2, 16, 32, 64, 128):
            for rows in (1, 2, 17, 138, 512):
                q = rows * ranks
                sw = O.moe_ready_swiglu_region_bytes(q * 512, experts)
                dp = O.moe_ready_dispatch_region_bytes(q * 512, ranks, experts)
                assert sw % 512 == 0 and dp % 512 == 0 and sw >= q * 512 and dp >= q * 512
                assert experts * 64 <= sw and (ranks * experts * 4 + 63) // 64 * 64 + experts * 64 <= dp


def test_ffn_end_to_end_small_is_self_consistent():
    """The chain on a tiny shape: combine of GMM2 rows equals a per-token loop."""
    rng = np.random.default_rng(9)
    t, k, n, e, topk = 12, 256, 512, 4, 2
    x = W.normal_bf16((t, k), 1)
    idx = np.stack([rng.permutation(e)[:topk] for _ in range(t)]).astype(np.int32)
    p = rng.random((t, topk)).astype(np.float32); p /= p.sum(1, keepdims=True)
    w1 = [O.mx_quant(rng.standard_normal((n, k)).astype(np.float32) * 0.05, "E4M3", "lut") for _ in range(e)]
    w2 = [O.mx_quant(rng.standard_normal((k, n // 2)).astype(np.float32) * 0.05, "E4M3", "lut") for _ in range(e)]
    w1q, w1s = np.stack([a for a, _ in w1]), np.stack([b for _, b in w1])
    w2q, w2s = np.stack([a for a, _ in w2]), np.stack([b for _, b in w2])
    out, st = O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s, stages=True)
    assert out.shape == (t, k) and st["counts"].sum() == t * topk
    xq, xs = O.mx_quant_bf16(x)
    acc = np.zeros((t, k), dtype=np.float32)
    for tok in range(t):
        for kk in range(topk):
            ex = idx[tok, kk]
            h = O.f32_to_bf16_bits(O.mx_gemm_f32(xq[tok:tok + 1], xs[tok:tok + 1], w1q[ex], w1s[ex]))
            a = O.swiglu_bf16(h)
            qa, sa = O.mx_quant_bf16(a)
            y = O.bf16_round(O.mx_gemm_f32(qa, sa, w2q[ex], w2s[ex]))
            term = (y[0] * p[tok, kk]).astype(np.float32)
            acc[tok] = term if kk == 0 else (acc[tok] + term).astype(np.float32)
    # per-row GEMV vs batched sgemm may differ in the last fp32 bit before the bf16 rounding
    ok, err, eb = O.verify_bf16(out, acc, k)
    assert ok and err == 0
    assert np.mean(out != O.f32_to_bf16_bits(acc)) < 0.02


def test_file_layouts_of_operands_by_explicit_indexing():
    """The [K, R] / [K/64, R, 2] file orientation, checked element by element with the index arithmetic of the
    generator written out (gen_data_mxfp8_mmrs.py:314-330: scale (r, kb) lands at ((kb // 2) * R + r) * 2 + kb % 2),
    and through the golden's own dequantisation of that orientation (:349-352: scales repeated 32 times along K)."""
    rng = np.random.default_rng(21)
    r, k = 5, 192
    codes, scales = _rand_mx(rng, r, k)
    fc, fs = O.to_file_layout(codes, scales, True)
    assert fc.shape == (k, r) and fs.shape == (k // 64, r, 2)
    flat = fs.reshape(-1)
    for i in range(r):
        for kk in range(k):
            assert fc[kk, i] == codes[i, kk]
            kb = kk // 32
            assert flat[((kb // 2) * r + i) * 2 + kb % 2] == scales[i, kb]
    # golden-style dequantisation of the [K, R] orientation: scale matrix [K/32, R] repeated along K
    smat = np.zeros((k // 32, r), dtype=np.uint8)
    for kb in range(k // 32):
        smat[kb] = fs[kb // 2, :, kb % 2]
    deq_file = O.decode(fc, "E4M3") * np.exp2(np.repeat(smat.astype(np.float64) - 127, 32, axis=0))
    assert np.array_equal(deq_file.astype(np.float32), O.mx_dequant(codes, scales).T)
    # stored-transposed orientation: the same bytes, and both directions invert
    nc, ns = O.to_file_layout(codes, scales, False)
    assert np.array_equal(nc, codes) and np.array_equal(ns.reshape(r, -1), scales[:, :k // 32])
    for trans in (False, True):
        c2, s2 = O.from_file_layout(*O.to_file_layout(codes, scales, trans), trans)
        assert np.array_equal(c2, codes) and np.array_equal(s2, scales[:, :k // 32])


def test_fp4_file_layouts_by_explicit_indexing():
    """FP4 bytes of the K-slow orientation: code (r, k) sits in byte [k, r // 2], low nibble for even r
    (gen_data_fp4_mx_alltoallv_gmm.py:522-545 applied to the transposed matrix, :586-620)."""
    rng = np.random.default_rng(22)
    r, k = 7, 128
    codes = rng.integers(0, 16, size=(r, k), dtype=np.uint8)
    scales = rng.integers(100, 140, size=(r, k // 32), dtype=np.uint8)
    fb, fs = O.to_file_layout_fp4(codes, scales, True)
    assert fb.shape == (k, (r + 1) // 2) and fs.shape == (k // 64, r, 2)
    for i in range(r):
        for kk in range(k):
            byte = int(fb[kk, i // 2])
            assert ((byte >> 4) if i % 2 else (byte & 15)) == codes[i, kk]
            kb = kk // 32
            assert fs[kb // 2, i, kb % 2] == scales[i, kb]
    assert np.all(fb[:, -1] >> 4 == 0)                       # the odd row count leaves the last high nibble empty
    nb, ns = O.to_file_layout_fp4(codes, scales, False)
    assert np.array_equal(nb, O.pack_fp4(codes)) and np.array_equal(ns.reshape(r, -1), scales)
