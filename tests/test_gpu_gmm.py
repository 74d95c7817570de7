"""Grouped matmul over ragged expert groups, with and without the fused SwiGLU + requant."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import dev, host, close_bf16, hooked_library, hooks_lib

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _hooked(request):
    """Tests that pin a tile shape run the package's front end on the test build of the library (the only one with
    that switch).  The cases of a tile matrix that leave the choice to the library (tile = None) run on the product
    library itself: its object file is a compilation of its own, and the hand-scheduled kernels depend on what the
    register allocator did in that very compilation."""
    params = getattr(getattr(request.node, "callspec", None), "params", {})
    if "tile" in params and params["tile"] is None:
        yield
        return
    with hooked_library():
        yield


def _weights(rng, g, n, k, std=0.05, fmt="E4M3"):
    qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) * std), fmt, "lut") for _ in range(g)]
    return np.stack([q for q, _ in qs]), np.stack([s for _, s in qs])


@pytest.mark.parametrize("tile", [None, (256, 256, 4), (256, 256, 5), (256, 128, 5), (256, 256, 8), (256, 128, 4), (256, 128, 8), (256, 64, 4), (128, 128, 4)])
@pytest.mark.parametrize("counts", [[5, 0, 300, 1, 0, 257, 64], [0, 0, 7], [512], [1] * 9])
def test_gmm_fp8_ragged_groups(tile, counts):
    from catccos_amd import ops, _lib
    if tile:
        hooks_lib().cmx_debug_force_tile(*tile)
    rng = np.random.default_rng(sum(counts))
    n, k = 320, 256
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m + 3, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=1.0)
    c = torch.full((m + 3, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k, c=c)
    got = host(c)
    gold = O.mx_gmm_f32(aq[:m], asc[:m], wq, ws, counts)
    bad, worst = close_bf16(got[:m], gold)
    assert bad == 0, (bad, worst)
    assert np.all(O.bf16_bits_to_f32(got[m:]) == 7.0)          # rows past the groups stay untouched


@pytest.mark.parametrize("tile", [None, (256, 256, 5), (256, 128, 5), (256, 256, 8), (128, 128, 4)])
def test_gmm_many_ragged_groups_every_row(tile):
    """43 groups whose sizes mix empty, whole-tile and ragged cases (equal remainders included): the ragged last
    m-tiles are numbered apart from the full ones and sorted by size, and every row must still be computed
    exactly once with its own group's weights."""
    from catccos_amd import ops, _lib
    if tile:
        hooks_lib().cmx_debug_force_tile(*tile)
    rng = np.random.default_rng(77)
    counts = [int(c) for c in rng.integers(0, 700, size=36)] + [256, 512, 0, 128, 128, 1, 255]
    n, k = 256, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=1.0)
    c = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k, c=c)
    gold = O.mx_gmm_f32(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(c), gold)
    assert bad == 0, (bad, worst)
    wq, ws = _weights(rng, len(counts), n, k, std=0.06)     # gate values of order 1: SiLU stays well conditioned
    codes, scales, act = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k,
                                                 want_bf16=True)
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    wq2, ws2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
    assert np.array_equal(host(scales), ws2) and np.array_equal(host(codes), wq2)


@pytest.mark.parametrize("fmt,k,waves", [("E4M3", 512, 4), ("E4M3", 1536, 4), ("E2M1", 512, 4), ("E2M1", 1024, 4), ("E2M1", 1536, 4),
                                         ("E2M1", 512, 5), ("E2M1", 1536, 5)])
def test_more_tiles_than_workgroups_every_row(fmt, k, waves):
    """Enough tiles (about 300 of 256 x 256) that the persistent kernels, one workgroup per CU, walk on to a second
    tile: the load stream crosses the tile boundary, the next tile comes from the per-XCD counters (4 x 1 wavefronts) or
    a fixed stride (2 x 2), and every row of every group must still come out right, with the rows past the groups
    untouched."""
    from catccos_amd import ops, _lib
    hooks_lib().cmx_debug_force_tile(256, 256, waves)
    rng = np.random.default_rng(91)
    counts = [int(c) for c in rng.integers(0, 700, size=36)] + [256, 512, 0, 128, 1, 255]
    n = 1024
    m = sum(counts)
    if fmt == "E2M1":
        aq, asc = O.mx_quant(rng.uniform(-2, 2, (m + 3, k)).astype(np.float32), "E2M1")
        qs = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in counts]
        pack = O.pack_fp4
    else:
        aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m + 3, k)).astype(np.float32)))
        qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32))) for _ in counts]
        pack = lambda x: x
    wq, ws = np.stack([q for q, _ in qs]), np.stack([s_ for _, s_ in qs])
    c = torch.full((m + 3, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(pack(aq)), dev(asc), dev(pack(wq)), dev(ws), dev(np.array(counts, dtype=np.int32)), k, fmt, "bf16", c=c)
    got = host(c)
    bad, worst = close_bf16(got[:m], O.mx_gmm_f32(aq[:m], asc[:m], wq, ws, counts, fmt, fmt))
    assert bad == 0, (bad, worst)
    assert np.all(O.bf16_bits_to_f32(got[m:]) == 7.0)


@pytest.mark.parametrize("waves", [4, 5])
def test_swiglu_requant_more_tiles_than_workgroups(waves):
    """The fused GMM1 epilogue on about 300 tiles: the persistent kernels (2 x 2 and 4 x 1 wavefronts) go through
    the epilogue and on to a next tile."""
    from catccos_amd import ops, _lib
    hooks_lib().cmx_debug_force_tile(256, 256, waves)
    rng = np.random.default_rng(92)
    counts = [int(c) for c in rng.integers(0, 700, size=36)] + [256, 512, 0, 128, 1, 255]
    n, k = 1024, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=0.06)
    codes, scales, act = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k,
                                                 want_bf16=True)
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    wq2, ws2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
    assert np.array_equal(host(scales), ws2) and np.array_equal(host(codes), wq2)
    codes_p, scales_p = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k)[:2]
    assert torch.equal(codes_p, codes) and torch.equal(scales_p, scales)        # same without the bf16 output


@pytest.mark.parametrize("fmt", ["E4M3", "E2M1"])
def test_groups_of_many_m_tiles_every_row(fmt):
    """Groups of 3 to 12 m-tiles (bands of eight m-tiles plus a rest of 1, 3, 4 or 6): the persistent 2 x 2 kernels prefetch
    each workgroup's share of the weight panel that the m-tiles of a band have in common, rows congruent to the tile's
    position in the band, and walk their XCD's tiles in fixed strides.  Every row of every group against the oracle."""
    from catccos_amd import ops
    rng = np.random.default_rng(93)
    counts = [2304, 0, 2048, 1300, 768, 1, 3000, 2815, 513]
    n, k = 512, 1024
    m = sum(counts)
    if fmt == "E2M1":
        aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
        qs = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in counts]
        pack = O.pack_fp4
    else:
        aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
        qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32))) for _ in counts]
        pack = lambda x: x
    wq, ws = np.stack([q for q, _ in qs]), np.stack([s_ for _, s_ in qs])
    c = ops.mx_gmm(dev(pack(aq)), dev(asc), dev(pack(wq)), dev(ws), dev(np.array(counts, dtype=np.int32)), k, fmt, "bf16")
    bad, worst = close_bf16(host(c), O.mx_gmm_f32(aq, asc, wq, ws, counts, fmt, fmt))
    assert bad == 0, (bad, worst)


def test_swiglu_requant_groups_of_many_m_tiles():
    """The fused GMM1 epilogue on the same kind of groups: the 2 x 2 kernel (weight-panel prefetch, strided walk) and the
    4 x 1 kernel (neither) give the same codes and scales, and both requantise their own bf16 values exactly."""
    from catccos_amd import ops
    rng = np.random.default_rng(94)
    counts = [2304, 0, 2048, 1300, 768, 1, 3000, 2815, 513]
    n, k = 1024, 1024
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=0.06)
    args = (dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k)
    lib = hooks_lib()
    outs = {}
    for waves in (4, 5):
        lib.cmx_debug_force_tile(256, 256, waves)
        codes, scales, act = ops.mx_gmm_swiglu_quant(*args, want_bf16=True)
        wq2, ws2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
        assert np.array_equal(host(scales), ws2) and np.array_equal(host(codes), wq2), waves
        outs[waves] = ops.mx_gmm_swiglu_quant(*args)[:2]
        assert torch.equal(outs[waves][0], codes) and torch.equal(outs[waves][1], scales), waves
    assert torch.equal(outs[4][0], outs[5][0]) and torch.equal(outs[4][1], outs[5][1])
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("tile", [None, (256, 128, 5), (128, 128, 4)])
def test_group_sizes_that_overrun_the_buffers_are_cut_off(tile):
    """The sizes are device data the host cannot check: rows past m_total are dropped group by group and negative
    sizes count as zero, so the kernels never leave the caller's buffers."""
    from catccos_amd import ops, _lib
    if tile:
        hooks_lib().cmx_debug_force_tile(*tile)
    rng = np.random.default_rng(41)
    n, k, m = 192, 512, 400
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, 4, n, k, std=1.0)
    claimed = np.array([300, -5, 300, 1 << 30], dtype=np.int32)          # only 300 + 100 rows exist
    c = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), dev(claimed), k, c=c)
    gold = O.mx_gmm_f32(aq, asc, wq, ws, [300, 0, 100, 0])
    bad, worst = close_bf16(host(c), gold)
    assert bad == 0, (bad, worst)


@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
def test_groups_about_one_tile_long(fmt):
    """Average group size between 128 and 512 rows with the default dispatch (256-row tiles, 4 x 1 wavefronts):
    remainders of 1, 64, 65, 128 and 129 rows past whole tiles, groups below and above one tile."""
    from catccos_amd import ops
    rng = np.random.default_rng(53)
    counts = [257, 256, 100, 320, 384, 385, 0, 250, 513, 129, 64, 300]
    assert 128 < sum(counts) / len(counts) < 512
    n, k = 320, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m + 5, k)).astype(np.float32)), fmt)
    qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32)), fmt, "rne") for _ in counts]
    wq, ws = np.stack([q for q, _ in qs]), np.stack([s_ for _, s_ in qs])
    c = torch.full((m + 5, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k, fmt, c=c)
    got = host(c)
    bad, worst = close_bf16(got[:m], O.mx_gmm_f32(aq[:m], asc[:m], wq, ws, counts, fmt, fmt))
    assert bad == 0, (bad, worst)
    assert np.all(O.bf16_bits_to_f32(got[m:]) == 7.0)


def test_swiglu_requant_with_groups_about_one_tile_long():
    from catccos_amd import ops
    rng = np.random.default_rng(54)
    counts = [257, 256, 100, 320, 384, 385, 0, 250, 513, 129, 64, 300]
    n, k = 512, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=0.06)
    codes, scales, act = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k,
                                                 want_bf16=True)
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    wq2, ws2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
    assert np.array_equal(host(scales), ws2) and np.array_equal(host(codes), wq2)


@pytest.mark.parametrize("tile", [None, (256, 256, 4), (256, 256, 5), (256, 256, 8)])
@pytest.mark.parametrize("k", [512, 1536, 640])
def test_gmm_fp4_ragged_groups(tile, k):
    from catccos_amd import ops, _lib
    if tile:
        hooks_lib().cmx_debug_force_tile(*tile)
    rng = np.random.default_rng(3)
    counts = [40, 0, 129, 300]
    n = 256
    m = sum(counts)
    aq, asc = O.mx_quant(rng.uniform(-2, 2, (m, k)).astype(np.float32), "E2M1")
    asc = (asc.astype(np.int32) + rng.integers(-2, 3, asc.shape)).astype(np.uint8)      # no two neighbouring blocks alike
    ws_ = [O.mx_quant(rng.uniform(-2, 2, (n, k)).astype(np.float32), "E2M1") for _ in counts]
    wq, ws = np.stack([q for q, _ in ws_]), np.stack([s for _, s in ws_])
    ws = (ws.astype(np.int32) + rng.integers(-2, 3, ws.shape)).astype(np.uint8)
    c = ops.mx_gmm(dev(O.pack_fp4(aq)), dev(asc), dev(O.pack_fp4(wq)), dev(ws), dev(np.array(counts, dtype=np.int32)), k,
                   "E2M1", "fp16")
    gold = O.mx_gmm_f32(aq, asc, wq, ws, counts, "E2M1", "E2M1")
    assert np.allclose(host(c).astype(np.float64), gold, rtol=2e-3, atol=5e-2)


@pytest.mark.parametrize("tile", [None, (256, 256, 4), (256, 256, 5), (256, 128, 5), (256, 256, 8), (256, 128, 4), (256, 128, 8), (256, 64, 4), (128, 128, 4)])
def test_gmm1_swiglu_requant(tile):
    """h and act are within tolerance of the golden chain; the requantised codes and scales are
    bit-exact against the oracle quantizer applied to the kernel's own bf16 SwiGLU output."""
    from catccos_amd import ops, _lib
    if tile:
        hooks_lib().cmx_debug_force_tile(*tile)
    rng = np.random.default_rng(12)
    counts = [70, 0, 300, 3, 130]
    n, k = 512, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, std=0.06)
    codes, scales, act = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws),
                                                 dev(np.array(counts, dtype=np.int32)), k, want_bf16=True)
    h_g, act_g, q_g, s_g = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    act_bits = host(act)
    # gate and up are each rounded to bf16 before the product (+-2^-8 each) and the product is
    # rounded again, so a one-ulp flip of either input moves act by up to ~1.2%: rtol 2e-2 here
    bad, worst = close_bf16(act_bits, O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    wq2, ws2 = O.mx_quant_bf16(act_bits, "E4M3", "rne")
    assert np.array_equal(host(scales), ws2)
    assert np.array_equal(host(codes), wq2)
    # the kernels that do not write the bf16 activations (separate instantiations) produce the same codes and scales
    codes_p, scales_p = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(np.array(counts, dtype=np.int32)), k)[:2]
    assert torch.equal(codes_p, codes) and torch.equal(scales_p, scales)
    # end to end the dequantised activations stay within tolerance of the golden's
    deq = O.mx_dequant(host(codes), host(scales))
    deq_g = O.mx_dequant(q_g, s_g)
    # a flipped rounding decision moves an element by one E4M3 step (2^-3 relative), a flipped
    # block exponent by one step of the coarser grid: bound by a step of the row's largest value
    bound = 0.13 * np.abs(deq_g) + 2.0 ** -5 * np.abs(deq_g).max(axis=1, keepdims=True)
    assert np.all(np.abs(deq - deq_g) <= bound)


def test_config3_routing_shape_small_hidden():
    """Zipf-routed ragged groups with two empty experts (the config-3 generator at reduced K/N)."""
    from catccos_amd import ops
    idx = W.zipf_routing(1024, 16, 8, seed=3)
    counts = np.bincount(idx.reshape(-1), minlength=16).astype(np.int32)
    assert (counts == 0).sum() == 2 and counts.sum() == 8192
    rng = np.random.default_rng(4)
    n, k = 512, 256
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((8192, k)).astype(np.float32)))
    wq, ws = _weights(rng, 16, n, k, std=0.08)
    codes, scales, act = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), dev(counts), k, want_bf16=True)
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    wq2, ws2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
    assert np.array_equal(host(scales), ws2) and np.array_equal(host(codes), wq2)


@pytest.mark.parametrize("k", [96, 160, 32])
@pytest.mark.parametrize("fmt", ["E4M3", "E2M1"])
def test_gmm_odd_block_count_weight_scales_have_the_even_padded_pitch(k, fmt):
    """K / 32 odd: scale rows, of the weights too, are padded to an even count (what the quantizer and the reference's
    generators write), so every weight row after the first sits at a pitch of K/32 + 1 bytes."""
    from catccos_amd import ops
    rng = np.random.default_rng(k)
    counts = [3, 0, 70, 129]
    n, m = 192, sum(counts)
    mode = "lut" if fmt == "E2M1" else "rne"
    a, a_s = ops.mx_quant(dev(O.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))).view(torch.bfloat16), fmt, mode)
    wq, ws = [], []
    for _ in counts:                                        # weights straight from the library's own quantizer
        q, s = ops.mx_quant(dev(O.f32_to_bf16_bits(rng.standard_normal((n, k)).astype(np.float32))).view(torch.bfloat16), fmt, "lut")
        wq.append(q)
        ws.append(s)
    w, w_s = torch.stack(wq).contiguous(), torch.stack(ws).contiguous()
    assert w_s.shape[2] == O.scale_cols(k) == k // 32 + 1
    c = ops.mx_gmm(a, a_s, w, w_s, dev(np.array(counts, dtype=np.int32)), k, fmt)
    un = (lambda t: O.unpack_fp4(host(t))) if fmt == "E2M1" else host
    gold = O.mx_gmm_f32(un(a), host(a_s), np.stack([un(q) for q in wq]), host(w_s), counts, fmt, fmt)
    bad, worst = close_bf16(host(c), gold, atol=5e-2 if fmt == "E2M1" else 1e-2)
    assert bad == 0, (bad, worst)
    if fmt == "E4M3" and n % 64 == 0:
        codes, scales, act = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, dev(np.array(counts, dtype=np.int32)), k, want_bf16=True)
        q2, s2 = O.mx_quant_bf16(host(act), "E4M3", "rne")
        assert np.array_equal(host(codes), q2) and np.array_equal(host(scales), s2)
        _, act_g, _, _ = O.gmm1_swiglu_quant(host(a), host(a_s), host(w), host(w_s), counts)
        bad, worst = close_bf16(host(act), O.bf16_bits_to_f32(act_g), rtol=2e-2)
        assert bad == 0, (bad, worst)
