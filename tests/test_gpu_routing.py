"""Bit-exact parity of the routing sort, the fused quantise+scatter and the weighted combine."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import dev, host, bf16_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens,experts,top_k,seed", [(1, 4, 1, 0), (7, 5, 3, 1), (512, 16, 6, 2), (1000, 256, 8, 3),
                                                       (8192, 256, 8, 4), (4096, 16, 8, 5), (333, 1000, 4, 6)])
def test_sort_matches_stable_argsort(tokens, experts, top_k, seed):
    from catccos_amd import ops
    rng = np.random.default_rng(seed)
    if experts == 16 and top_k == 8:
        idx = W.zipf_routing(tokens, experts, top_k, seed)
    else:
        idx = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    s2s, inv, counts = ops.moe_init_routing(dev(idx), experts)
    w_s2s, w_inv, w_counts = O.moe_init_routing(idx, experts)
    assert np.array_equal(host(counts), w_counts)
    assert np.array_equal(host(s2s), w_s2s)
    assert np.array_equal(host(inv), w_inv)


def test_sort_all_routes_to_one_expert_and_repeats():
    from catccos_amd import ops
    idx = np.full((700, 3), 2, dtype=np.int32)          # duplicates inside a token are legal keys for the sort
    s2s, inv, counts = ops.moe_init_routing(dev(idx), 4)
    assert np.array_equal(host(s2s), np.arange(2100)) and host(counts).tolist() == [0, 0, 2100, 0]
    bal = O.balanced_expert_idx(512, 16, 6, 1)[0]
    s2s, inv, counts = ops.moe_init_routing(dev(bal), 16)
    assert host(counts).tolist() == [192] * 16
    assert np.array_equal(host(s2s), O.moe_init_routing(bal, 16)[0])


@pytest.mark.parametrize("packed", [False, True])
def test_quant_scatter_bit_exact(packed):
    from catccos_amd import ops
    tokens, k, top_k, experts = 300, 512, 4, 8
    rng = np.random.default_rng(7)
    xb = W.activations_with_outliers(tokens, k, seed=8)
    idx = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    _, inv, _ = O.moe_init_routing(idx, experts)
    want = O.quant_scatter_packed(xb, inv, top_k)
    if packed:
        buf = ops.quant_scatter(bf16_dev(xb), dev(inv), top_k, packed=True)
        assert np.array_equal(host(buf), want)
    else:
        codes, scales = ops.quant_scatter(bf16_dev(xb), dev(inv), top_k)
        assert np.array_equal(host(codes), want[:, :k]) and np.array_equal(host(scales), want[:, k:k + k // 32])


@pytest.mark.parametrize("k", [64, 96, 480, 512, 4064])
def test_quant_scatter_packed_rows_touch_nothing_else(k):
    """The packed wire layout (scale bytes behind the codes of the same row): every byte of the buffer is the oracle's,
    pad bytes included, and the bytes in front of the first and behind the last row keep their fill.  k = 96 is the case
    whose packed row (128 bytes) equals the scale row rounded up to a whole 128-byte line."""
    from catccos_amd import ops
    tokens, top_k, experts, guard = 40, 3, 6, 4
    rng = np.random.default_rng(k)
    xb = W.activations_with_outliers(tokens, k, seed=k + 1)
    idx = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    _, inv, _ = O.moe_init_routing(idx, experts)
    want = O.quant_scatter_packed(xb, inv, top_k)
    rows, rb = want.shape
    assert rb == O.packed_row_bytes(k)
    whole = torch.full((rows + 2 * guard, rb), 0xA5, dtype=torch.uint8, device="cuda")
    mid = whole[guard:guard + rows]
    mid.zero_()
    ops.quant_scatter(bf16_dev(xb), dev(inv), top_k, packed=True, out=mid)
    got = host(whole)
    assert np.array_equal(got[guard:guard + rows], want)
    assert np.all(got[:guard] == 0xA5) and np.all(got[guard + rows:] == 0xA5)


@pytest.mark.parametrize("k", [512, 7168, 96])
def test_quant_scatter_non_finite_tokens_equal_the_quantizer(k):
    """Tokens with Inf / NaN elements through both scatter kernels (k = 96: scale rows that are not 16-byte aligned take the
    general kernel) give the rows the stand-alone quantizer and the oracle give."""
    from catccos_amd import ops
    from tests.test_gpu_quant import _with_non_finite
    tokens, top_k = 24, 3
    xb = _with_non_finite(tokens, k, seed=k)
    rng = np.random.default_rng(k)
    inv = rng.permutation(tokens * top_k).astype(np.int32)
    codes, scales = ops.quant_scatter(bf16_dev(xb), dev(inv), top_k)
    q, s = O.mx_quant_bf16(xb)
    got_c, got_s = host(codes), host(scales)
    nsc = s.shape[1]
    for t in range(tokens):
        for r in range(top_k):
            d = inv[t * top_k + r]
            assert np.array_equal(got_c[d], q[t]), (t, r)
            assert np.array_equal(got_s[d, :nsc], s[t]), (t, r)


def test_quant_scatter_skips_negative_destinations():
    from catccos_amd import ops
    xb = W.activations_with_outliers(8, 64, seed=9)
    inv = np.arange(16, dtype=np.int32)
    inv[3] = -1
    codes, scales = ops.quant_scatter(bf16_dev(xb), dev(inv), 2)
    q, s = O.mx_quant_bf16(xb)
    got = host(codes)
    assert np.all(got[3] == 0) and np.array_equal(got[2], q[1]) and np.array_equal(got[4], q[2])


@pytest.mark.parametrize("tokens,hidden,top_k", [(5, 64, 1), (33, 7168, 8), (100, 520, 6), (64, 2048, 3), (9, 100, 9)])
def test_combine_bit_exact(tokens, hidden, top_k):
    from catccos_amd import ops
    rng = np.random.default_rng(tokens)
    experts = max(top_k, 12)
    idx = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    _, inv, _ = O.moe_init_routing(idx, experts)
    pad = (-hidden) % 8                                  # rows must be 16-byte aligned: pitch rounded up
    y = W.normal_bf16((tokens * top_k, hidden + pad), seed=tokens + 1)
    p = rng.random((tokens, top_k)).astype(np.float32)
    p /= p.sum(1, keepdims=True)
    yd = bf16_dev(y)
    if pad == 0:
        out = host(ops.moe_token_unpermute(yd, dev(inv), dev(p)))
        assert np.array_equal(out, O.unpermute_combine(y, inv, p))
    else:
        from catccos_amd import _lib
        o = torch.zeros((tokens, hidden + pad), dtype=torch.bfloat16, device="cuda")
        inv_d, p_d = dev(inv), dev(p)
        _lib.check(_lib.load().cmx_moe_token_unpermute(yd.data_ptr(), hidden + pad, tokens * top_k, inv_d.data_ptr(),
                                                       p_d.data_ptr(), o.data_ptr(), hidden + pad, tokens, hidden,
                                                       top_k, torch.cuda.current_stream().cuda_stream))
        assert np.array_equal(host(o)[:, :hidden], O.unpermute_combine(y[:, :hidden], inv, p))


def test_combine_ignores_out_of_range_rows():
    from catccos_amd import ops
    y = W.normal_bf16((12, 64), seed=2)
    inv = np.arange(12, dtype=np.int32)
    inv[0] = 50
    inv[7] = -3
    p = np.random.default_rng(3).random((4, 3)).astype(np.float32)
    out = host(ops.moe_token_unpermute(bf16_dev(y), dev(inv), dev(p)))
    assert np.array_equal(out, O.unpermute_combine(y, inv, p))
