"""Pre-tiled expert weights: the tiling pass against a restatement of the published layout, and the grouped matmuls
and the FFN chain on pre-tiled weights against the oracle and, bit for bit, against the same entry points on
row-major weights."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import dev, host, bf16_dev, close_bf16, hooked_library, hooks_lib

pytestmark = pytest.mark.gpu

# tile heights of the kernel behind the pre-tiled entry points: None leaves the choice to the product library (288 rows
# for groups that average less than 1024 rows, else 256); the others pin it on the test build of the library
TILE_HEIGHTS = [None, 256, 288]


@pytest.fixture(autouse=True)
def _tile_height(request):
    params = getattr(getattr(request.node, "callspec", None), "params", {})
    tm = params.get("tm")
    if tm is None:
        yield
        return
    with hooked_library():
        hooks_lib().cmx_debug_pretiled_tile_rows(tm)
        yield


def pretile_numpy(w: np.ndarray, pair_gate_up: bool) -> np.ndarray:
    """[G, n, k] -> the byte order include/catccos_mx.h publishes, written index by index:
    [group][256-row tile][128-byte slab][wavefront][step h][fragment f][register half][lane / 32][lane % 32][16]."""
    g, n, k = w.shape
    if pair_gate_up:
        hn = n // 2
        tiles = -(-hn // 128)
        t, ww, f, l = np.meshgrid(np.arange(tiles), np.arange(4), np.arange(2), np.arange(32), indexing="ij")
        rows = np.minimum(t * 128 + ww * 32 + l, hn - 1) + f * hn
    else:
        tiles = -(-n // 256)
        t, ww, f, l = np.meshgrid(np.arange(tiles), np.arange(4), np.arange(2), np.arange(32), indexing="ij")
        rows = np.minimum(t * 256 + ww * 64 + f * 32 + l, n - 1)
    s, h, half, lh = np.meshgrid(np.arange(k // 128), np.arange(2), np.arange(2), np.arange(2), indexing="ij")
    cols = s * 128 + h * 64 + half * 32 + lh * 16                                         # [slab, h, half, lh]
    out = np.empty((g, tiles, k // 128, 4, 2, 2, 2, 2, 32, 16), dtype=np.uint8)
    for ti in range(tiles):
        for wi in range(4):
            for fi in range(2):
                r = rows[ti, wi, fi]                                                      # [32]
                for si in range(k // 128):
                    for hi in range(2):
                        for ha in range(2):
                            for li in range(2):
                                c = cols[si, hi, ha, li]
                                out[:, ti, si, wi, hi, fi, ha, li] = w[:, r, c:c + 16]
    return out.reshape(-1)


@pytest.mark.parametrize("g,n,k,pair", [(3, 320, 512, False), (2, 640, 1024, True), (1, 256, 512, False), (2, 64, 512, True)])
def test_pretile_pass_writes_the_published_order(g, n, k, pair):
    from catccos_amd import ops, _lib
    rng = np.random.default_rng(n + k)
    w = rng.integers(0, 256, size=(g, n, k), dtype=np.uint8)
    t = ops.pretile_weights(dev(w), pair)
    want = pretile_numpy(w, pair)
    assert t.data.numel() == want.size == _lib.load().cmx_mx_pretiled_weight_bytes(g, n, k, int(pair))
    assert np.array_equal(host(t.data), want)


def _weights(rng, g, n, k, std, fmt="E4M3"):
    qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) * std), fmt, "lut") for _ in range(g)]
    return np.stack([q for q, _ in qs]), np.stack([s for _, s in qs])


@pytest.mark.parametrize("tm", TILE_HEIGHTS)
@pytest.mark.parametrize("fmt,out", [("E4M3", "bf16"), ("E5M2", "fp16")])
@pytest.mark.parametrize("counts", [[5, 0, 300, 1, 0, 257, 64], [0, 0, 7], [512], [1] * 9, [288, 289, 287, 0, 576]])
def test_gmm_on_pretiled_weights(tm, fmt, out, counts):
    from catccos_amd import ops
    rng = np.random.default_rng(sum(counts) + 1)
    n, k = 320, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m + 3, k)).astype(np.float32)), fmt)
    wq, ws = _weights(rng, len(counts), n, k, 1.0, fmt)
    cnt = dev(np.array(counts, dtype=np.int32))
    dt = torch.bfloat16 if out == "bf16" else torch.float16
    c = torch.full((m + 3, n), 7.0, dtype=dt, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), ops.pretile_weights(dev(wq), False), dev(ws), cnt, k, fmt, out, c=c)
    gold = O.mx_gmm_f32(aq[:m], asc[:m], wq, ws, counts, fmt, fmt)
    if out == "bf16":
        bad, worst = close_bf16(host(c)[:m], gold)
        assert bad == 0, (bad, worst)
    else:
        got = c[:m].float().cpu().numpy()
        assert np.all(np.abs(got - gold) <= 1e-2 + 1e-2 * np.abs(gold))
    assert bool((c[m:].float() == 7.0).all())                  # rows past the groups stay untouched
    c_rm = torch.full((m + 3, n), 7.0, dtype=dt, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k, fmt, out, c=c_rm)
    assert torch.equal(c.view(torch.int16), c_rm.view(torch.int16))


@pytest.mark.parametrize("tm", TILE_HEIGHTS)
def test_gmm1_and_gmm2_on_pretiled_weights_many_ragged_groups(tm):
    """43 groups (empty, whole-tile, ragged) at one weight tile per group: fewer tiles than workgroups, so every tile is
    cut into row parts that different workgroups compute; every row must still come out once, with the bits of the
    row-major kernels, and agree with the oracle."""
    from catccos_amd import ops
    rng = np.random.default_rng(78)
    counts = [int(c) for c in rng.integers(0, 700, size=36)] + [256, 512, 0, 128, 128, 1, 255]
    n, k = 256, 512
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    cnt = dev(np.array(counts, dtype=np.int32))
    wq, ws = _weights(rng, len(counts), n, k, 1.0)
    c = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.mx_gmm(dev(aq), dev(asc), ops.pretile_weights(dev(wq), False), dev(ws), cnt, k, c=c)
    bad, worst = close_bf16(host(c), O.mx_gmm_f32(aq, asc, wq, ws, counts))
    assert bad == 0, (bad, worst)
    assert torch.equal(c, ops.mx_gmm(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k))
    wq, ws = _weights(rng, len(counts), n, k, 0.06)       # gate values of order 1: SiLU stays well conditioned
    codes, scales, none = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), ops.pretile_weights(dev(wq), True), dev(ws), cnt, k)
    assert none is None
    # against the oracle through the bf16 values that the row-major instantiation with that output writes: those are
    # checked against the oracle's, and the codes and scales must be the oracle quantizer's image of them
    codes_r, scales_r, act_r = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k, want_bf16=True)
    _, act_g, _, _ = O.gmm1_swiglu_quant(aq, asc, wq, ws, counts)
    bad, worst = close_bf16(host(act_r), O.bf16_bits_to_f32(act_g), rtol=2e-2)
    assert bad == 0, (bad, worst)
    q2, s2 = O.mx_quant_bf16(host(act_r), "E4M3", "rne")
    assert np.array_equal(host(scales), s2) and np.array_equal(host(codes), q2)
    assert torch.equal(codes, codes_r) and torch.equal(scales, scales_r)


@pytest.mark.parametrize("tm", TILE_HEIGHTS)
@pytest.mark.parametrize("groups,n", [(60, 1280), (70, 1024)])
def test_pretiled_more_tiles_than_workgroups(tm, groups, n):
    """Several rounds of tiles per workgroup (tiles drawn from the per-XCD counters while the load streams of the
    previous tile are still running) and a partly filled last round, bit for bit against the row-major kernels on
    GPU-made operands; sampled rows against the oracle."""
    from catccos_amd import ops
    k = 1024
    g = torch.Generator(device="cuda")
    g.manual_seed(groups)
    counts_h = np.random.default_rng(groups).integers(120, 300, size=groups).astype(np.int32)
    m = int(counts_h.sum())
    a, a_s = ops.mx_quant(torch.randn((m, k), generator=g, device="cuda").to(torch.bfloat16), "E4M3", "rne")
    w, w_s = ops.mx_quant((torch.randn((groups * n, k), generator=g, device="cuda") * 0.05).to(torch.bfloat16), "E4M3", "lut")
    w, w_s = w.view(groups, n, k), w_s.view(groups, n, -1)
    cnt = torch.from_numpy(counts_h).cuda()
    y = ops.mx_gmm(a, a_s, ops.pretile_weights(w, False), w_s, cnt, k)
    assert torch.equal(y, ops.mx_gmm(a, a_s, w, w_s, cnt, k))
    off = np.concatenate([[0], np.cumsum(counts_h)])
    for e in (0, groups // 2, groups - 1):
        rows = torch.arange(int(off[e]), int(off[e + 1]), device="cuda")
        gold = O.mx_gmm_f32(host(a[rows]), host(a_s[rows]), host(w[e:e + 1]), host(w_s[e:e + 1]), [len(rows)])
        bad, worst = close_bf16(host(y[rows]), gold)
        assert bad == 0, (e, bad, worst)
    c1, s1, _ = ops.mx_gmm_swiglu_quant(a, a_s, ops.pretile_weights(w, True), w_s, cnt, k)
    c2, s2, _ = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, k)
    assert torch.equal(c1, c2) and torch.equal(s1, s2)


def test_pretiled_entry_points_reject_what_the_kernel_cannot_take():
    from catccos_amd import ops, _lib
    rng = np.random.default_rng(5)
    counts = dev(np.array([40, 24], dtype=np.int32))
    with pytest.raises(ValueError):
        ops.pretile_weights(dev(rng.integers(0, 256, size=(2, 64, 256), dtype=np.uint8)), False)      # k % 512
    k, n = 512, 64
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((64, k)).astype(np.float32)))
    wq, ws = _weights(rng, 2, n, k, 1.0)
    tiled = ops.pretile_weights(dev(wq), False)
    with pytest.raises(_lib.CmxError, match="16-bit output"):
        ops.mx_gmm(dev(aq), dev(asc), tiled, dev(ws), counts, k, out="fp32")
    with pytest.raises(_lib.CmxError, match="8-bit element formats"):
        ops.mx_gmm(dev(aq), dev(asc), tiled, dev(ws), counts, k, fmt="E2M1")
    with pytest.raises(_lib.CmxError, match="16-byte aligned"):
        ops.mx_gmm(dev(aq), dev(np.pad(asc, ((0, 0), (0, 4))))[:, :k // 32], tiled, dev(ws), counts, k)     # scale pitch 20
    with pytest.raises(AssertionError):
        ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), tiled, dev(ws), counts, k)                              # tiled for the other matmul
    with pytest.raises(_lib.CmxError, match="act_bf16 must be NULL"):
        ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), ops.pretile_weights(dev(wq), True), dev(ws), counts, k, want_bf16=True)


def _ffn_inputs(tokens, k, n, experts, top_k, seed):
    rng = np.random.default_rng(seed)
    x = W.normal_bf16((tokens, k), seed)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, seed + 1)
    w1q, w1s = _weights(rng, experts, n, k, 1.0 / np.sqrt(k))
    w2q, w2s = _weights(rng, experts, k, n // 2, 1.0 / np.sqrt(n // 2))
    return x, idx, p, w1q, w1s, w2q, w2s


@pytest.mark.parametrize("tm", TILE_HEIGHTS)
@pytest.mark.parametrize("tokens,k,n,experts,top_k", [(64, 512, 1024, 16, 6), (777, 512, 2048, 8, 8)])
def test_ffn_on_pretiled_weights(tm, tokens, k, n, experts, top_k):
    from catccos_amd import ops
    x, idx, p, w1q, w1s, w2q, w2s = _ffn_inputs(tokens, k, n, experts, top_k, tokens)
    w1, w2 = dev(w1q), dev(w2q)
    ws = torch.full((ops.ffn_workspace_bytes(tokens, k, n, experts, top_k),), 0xA5, dtype=torch.uint8, device="cuda")
    out_t = ops.dispatch_ffn_combine(bf16_dev(x), dev(idx), dev(p), ops.pretile_weights(w1, True), dev(w1s),
                                     ops.pretile_weights(w2, False), dev(w2s), workspace=ws)
    gold = O.bf16_bits_to_f32(O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s))
    got = host(out_t)
    bad, worst = close_bf16(got, gold)
    assert bad <= got.size // 1000 and worst <= 5e-2, (bad, worst)
    out = ops.dispatch_ffn_combine(bf16_dev(x), dev(idx), dev(p), w1, dev(w1s), w2, dev(w2s))
    assert torch.equal(out_t, out)


def test_pretiled_ffn_rejects_bad_shapes():
    from catccos_amd import ops, _lib
    x, idx, p, w1q, w1s, w2q, w2s = _ffn_inputs(8, 512, 512, 4, 2, 3)          # N = 512: GMM2's K would be 256
    lib = _lib.load()
    ws = torch.empty(ops.ffn_workspace_bytes(8, 512, 512, 4, 2), dtype=torch.uint8, device="cuda")
    out = torch.empty((8, 512), dtype=torch.bfloat16, device="cuda")
    args = [t.data_ptr() for t in (bf16_dev(x), dev(idx), dev(p), dev(w1q), dev(w1s), dev(w2q), dev(w2s), out, ws)]
    assert lib.cmx_dispatch_ffn_combine_pretiled(None, *args, 8, 512, 512, 4, 2) == -1
    assert b"N % 1024" in lib.cmx_last_error()


def test_pretiled_long_groups_take_the_256_row_tile():
    """Groups that average 1024 rows or more: the product library picks the 256-row tile (several tiles per group and
    weight panel, the last one ragged); bit for bit against the row-major kernels."""
    from catccos_amd import ops
    k, n, groups = 512, 512, 3
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    counts_h = np.array([1500, 700, 1100], dtype=np.int32)
    m = int(counts_h.sum())
    a, a_s = ops.mx_quant(torch.randn((m, k), generator=g, device="cuda").to(torch.bfloat16), "E4M3", "rne")
    w, w_s = ops.mx_quant((torch.randn((groups * n, k), generator=g, device="cuda") * 0.05).to(torch.bfloat16), "E4M3", "lut")
    w, w_s = w.view(groups, n, k), w_s.view(groups, n, -1)
    cnt = torch.from_numpy(counts_h).cuda()
    assert torch.equal(ops.mx_gmm(a, a_s, ops.pretile_weights(w, False), w_s, cnt, k), ops.mx_gmm(a, a_s, w, w_s, cnt, k))
    c1, s1, _ = ops.mx_gmm_swiglu_quant(a, a_s, ops.pretile_weights(w, True), w_s, cnt, k)
    c2, s2, _ = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, k)
    assert torch.equal(c1, c2) and torch.equal(s1, s2)


@pytest.mark.parametrize("tm", TILE_HEIGHTS)
def test_pretiled_gmm_with_row_pitches(tm):
    """Activation, activation-scale and output rows at pitches larger than a row (what a caller's sub-view has): the bytes
    between the rows are neither read into the result nor written."""
    from catccos_amd import ops
    rng = np.random.default_rng(21)
    counts = [130, 0, 290, 33]
    n, k = 512, 1024
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    wq, ws = _weights(rng, len(counts), n, k, 1.0)
    a_big = torch.full((m, k + 64), 0x7F, dtype=torch.uint8, device="cuda")            # 0x7F: NaN codes in the padding
    a_big[:, :k] = dev(aq)
    s_big = torch.full((m, k // 32 + 16), 0xFF, dtype=torch.uint8, device="cuda")      # 0xFF: NaN scales in the padding
    s_big[:, :k // 32] = dev(asc)
    c_big = torch.full((m, n + 24), 7.0, dtype=torch.bfloat16, device="cuda")
    cnt = dev(np.array(counts, dtype=np.int32))
    ops.mx_gmm(a_big[:, :k], s_big[:, :k // 32], ops.pretile_weights(dev(wq), False), dev(ws), cnt, k, c=c_big[:, :n])
    bad, worst = close_bf16(host(c_big[:, :n].contiguous()), O.mx_gmm_f32(aq, asc, wq, ws, counts))
    assert bad == 0, (bad, worst)
    assert bool((c_big[:, n:].float() == 7.0).all())
    codes = torch.full((m, n // 2 + 32), 0xEE, dtype=torch.uint8, device="cuda")
    scales = torch.full((m, n // 64 + 6), 0xEE, dtype=torch.uint8, device="cuda")
    ops.mx_gmm_swiglu_quant(a_big[:, :k], s_big[:, :k // 32], ops.pretile_weights(dev(wq), True), dev(ws), cnt, k,
                            outs=(codes[:, :n // 2], scales[:, :n // 64]))
    c_r, s_r, _ = ops.mx_gmm_swiglu_quant(dev(aq), dev(asc), dev(wq), dev(ws), cnt, k)
    assert torch.equal(codes[:, :n // 2], c_r) and torch.equal(scales[:, :n // 64], s_r)
    assert bool((codes[:, n // 2:] == 0xEE).all()) and bool((scales[:, n // 64:] == 0xEE).all())


@pytest.mark.parametrize("tm", [256, 288])
def test_pretiled_seeded_sweep_matches_row_major_bits(tm):
    """Thirty seeded problems (group counts 1..40, group sizes from empty to several tiles, N ragged against the 256-row
    weight tile, K from one to six 512-byte blocks): both grouped matmuls on pre-tiled weights give the bits of the
    row-major entry points, whose parity with the oracle the other suites establish."""
    from catccos_amd import ops
    rng = np.random.default_rng(1000 + tm)
    g = torch.Generator(device="cuda")
    for case in range(30):
        groups = int(rng.integers(1, 41))
        kind = case % 3
        hi = (40, 300, 900)[kind]
        counts_h = rng.integers(0, hi + 1, size=groups).astype(np.int32)
        if counts_h.sum() == 0:
            counts_h[0] = 17
        m = int(counts_h.sum())
        k = 512 * int(rng.integers(1, 7))
        n = 64 * int(rng.integers(1, 21))
        g.manual_seed(case)
        a, a_s = ops.mx_quant(torch.randn((m, k), generator=g, device="cuda").to(torch.bfloat16), "E4M3", "rne")
        w, w_s = ops.mx_quant((torch.randn((groups * n, k), generator=g, device="cuda") * 0.06).to(torch.bfloat16), "E4M3", "lut")
        w, w_s = w.view(groups, n, k), w_s.view(groups, n, -1)
        cnt = torch.from_numpy(counts_h).cuda()
        what = (case, groups, m, n, k)
        y_t = ops.mx_gmm(a, a_s, ops.pretile_weights(w, False), w_s, cnt, k)
        assert torch.equal(y_t, ops.mx_gmm(a, a_s, w, w_s, cnt, k)), what
        c_t, s_t, _ = ops.mx_gmm_swiglu_quant(a, a_s, ops.pretile_weights(w, True), w_s, cnt, k)
        c_r, s_r, _ = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, k)
        assert torch.equal(c_t, c_r) and torch.equal(s_t, s_r), what
