"""The benchmark configurations 2-5 at their full sizes: sampled rows against the oracle plus properties that
do not depend on the size (exact scale linearity, row-permutation equivariance, gate-weight linearity).
Inputs are generated and quantised on the GPU; only the sampled rows travel to the host for the oracle."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import host, close_bf16

pytestmark = pytest.mark.gpu


def _gpu_mx(shape, seed, std=1.0, fmt="E4M3", mode="rne"):
    from catccos_amd import ops
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    x = (torch.randn(shape, generator=g, device="cuda") * std).to(torch.bfloat16)
    return ops.mx_quant(x, fmt, mode)


def _np(t):
    return t.cpu().numpy()


def _assert_rows_follow(got_bits, want_bits, what):
    """bf16 results (as int16 bit patterns) of the same rows computed in another place of the schedule.  The sums of a
    row do not depend on where its tile runs, so they are equal bit for bit -- except in tiles whose K range the
    schedule splits between two workgroups (the last, partly filled round of a launch), where the two partial sums
    are added in fp32 and the bf16 result may move by one unit in the last place."""
    if torch.equal(got_bits, want_bits):
        return
    g = got_bits.view(torch.bfloat16).float()
    w = want_bits.view(torch.bfloat16).float()
    tol = torch.maximum(g.abs(), w.abs()) * 2.0 ** -7 + 1e-30
    assert bool(((g - w).abs() <= tol).all()), what
    assert float((got_bits != want_bits).float().mean()) < 0.02, what


def test_config2_dense_full_size():
    from catccos_amd import ops
    M, N, K = 8192, 4096, 7168
    a, a_s = _gpu_mx((M, K), 21)
    b, b_s = _gpu_mx((N, K), 22)
    c = ops.mx_gemm(a, a_s, b, b_s, K)
    rows = np.array([0, 1, 255, 256, 257, 4095, 4096, 8190, 8191] + list(np.random.default_rng(0).integers(0, M, 23)))
    gold = O.mx_gemm_f32(_np(a[rows]), _np(a_s[rows]), _np(b), _np(b_s))
    bad, worst = close_bf16(host(c[rows]), gold)
    assert bad == 0, (bad, worst)
    # The reference judges this operator by its double-golden rule (fp32 golden + the same product rounded to bf16).
    # Its mean-error, RMSE and bias terms are checked as they stand.  Its maximum-relative-error term divides by
    # |gold| + 1e-7, so among the 33 million outputs of this size the few whose golden value is nearly zero fail it
    # for ANY fp32-accumulating kernel (an absolute error of 1e-5 on |gold| = 1e-4 is already 10 %); here it is
    # applied to the outputs with |gold| >= 1, and as it stands at the reference's own test shapes (tests/test_gpu_gemm.py).
    got = host(c[rows])
    _, r_max, r_mean, r_rmse, eb = O.verify_double_golden_bf16(got, gold, O.f32_to_bf16_bits(gold))
    assert r_mean < 2 and r_rmse < 2 and eb <= 2.0 ** -7, (r_max, r_mean, r_rmse, eb)
    big = np.abs(gold) >= 1.0
    ok, r_max, *_ = O.verify_double_golden_bf16(got[big], gold[big], O.f32_to_bf16_bits(gold[big]))
    assert ok, r_max
    # one more on every activation scale doubles every product and every partial sum: the bf16 result doubles exactly
    c2 = ops.mx_gemm(a, a_s + 1, b, b_s, K)
    assert torch.equal(c2.float(), c.float() * 2)
    # permuting activation rows permutes result rows bit for bit (a row's sums do not depend on its tile)
    perm = torch.randperm(M, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
    cp = ops.mx_gemm(a[perm].contiguous(), a_s[perm].contiguous(), b, b_s, K)
    assert torch.equal(cp, c[perm])


def test_config3_gmm1_swiglu_requant_full_size():
    from catccos_amd import ops
    E, T, TOPK, K, N = 16, 4096, 8, 7168, 4096
    idx = W.zipf_routing(T, E, TOPK, 3)
    counts = np.bincount(idx.reshape(-1), minlength=E).astype(np.int32)
    rows = int(counts.sum())
    a, a_s = _gpu_mx((rows, K), 31)
    w = torch.empty((E, N, K), dtype=torch.uint8, device="cuda")
    w_s = torch.empty((E, N, K // 32), dtype=torch.uint8, device="cuda")
    for e in range(E):
        w[e], w_s[e] = _gpu_mx((N, K), 100 + e, std=0.02, mode="lut")
    cnt = torch.from_numpy(counts).cuda()
    codes, scales, _ = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, K)
    # The instantiation that also writes the bf16 SwiGLU output must give the same codes and scales on every row,
    # and those must be, bit for bit, what the oracle quantizer makes of that bf16 output (all 32 768 rows, in
    # chunks to bound the host memory); the stand-alone HIP quantizer must agree as well.
    codes2, scales2, act = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, K, want_bf16=True)
    assert torch.equal(codes, codes2) and torch.equal(scales, scales2)
    hq, hs = ops.mx_quant(act, "E4M3", "rne")
    assert torch.equal(hq, codes) and torch.equal(hs, scales)
    for r0 in range(0, rows, 4096):
        r1 = min(rows, r0 + 4096)
        oq, osc = O.mx_quant_bf16(host(act[r0:r1]), "E4M3", "rne")
        assert np.array_equal(oq, _np(codes[r0:r1])), (r0, r1)
        assert np.array_equal(osc, _np(scales[r0:r1])), (r0, r1)
    off = np.concatenate([[0], np.cumsum(counts)])
    rng = np.random.default_rng(1)
    for e in [int(np.argmax(counts)), int(np.argmin(np.where(counts > 0, counts, 1 << 30))), 5]:
        if counts[e] == 0:
            continue
        pick = np.unique(np.concatenate([[0, counts[e] - 1], rng.integers(0, counts[e], 6)])) + off[e]
        _, gact, gq, gs = O.gmm1_swiglu_quant(_np(a[pick]), _np(a_s[pick]), _np(w[e:e + 1]), _np(w_s[e:e + 1]), [len(pick)])
        deq, deq_g = O.mx_dequant(_np(codes[pick]), _np(scales[pick])), O.mx_dequant(gq, gs)
        bound = 0.13 * np.abs(deq_g) + 2.0 ** -5 * np.abs(deq_g).max(axis=1, keepdims=True) + 1e-9
        assert np.all(np.abs(deq - deq_g) <= bound), e
        # the bf16 SwiGLU output itself against the golden chain
        bad, worst = close_bf16(host(act[pick]), O.bf16_bits_to_f32(gact), rtol=2e-2, atol=1e-3)
        assert bad == 0, (e, bad, worst)
    # every scale byte is a legal E8M0 value and no code is the E4M3 NaN pattern
    assert int((codes & 0x7F).eq(0x7F).sum()) == 0
    # group-order equivariance: the same rows as groups in reverse expert order give the same codes per row
    order = list(range(E - 1, -1, -1))
    src = torch.cat([torch.arange(off[e], off[e + 1], device="cuda") for e in order])
    codes_r, scales_r, _ = ops.mx_gmm_swiglu_quant(a[src].contiguous(), a_s[src].contiguous(), w[order].contiguous(),
                                                  w_s[order].contiguous(), torch.from_numpy(counts[order].copy()).cuda(), K)
    assert torch.equal(codes_r, codes[src]) and torch.equal(scales_r, scales[src])


def test_config5_fp4_gmm_full_size():
    from catccos_amd import ops
    E, T, K, N = 32, 8192, 7168, 4096
    idx = W.zipf_routing(T, E, 8, 8)
    counts = np.bincount(idx.reshape(-1), minlength=E).astype(np.int32)
    rows = int(counts.sum())
    g = torch.Generator(device="cuda")
    g.manual_seed(51)
    a, a_s = ops.mx_quant((torch.rand((rows, K), generator=g, device="cuda") * 4 - 2).to(torch.bfloat16), "E2M1", "lut")
    w = torch.empty((E, N, K // 2), dtype=torch.uint8, device="cuda")
    w_s = torch.empty((E, N, K // 32), dtype=torch.uint8, device="cuda")
    for e in range(E):
        w[e], w_s[e] = ops.mx_quant((torch.rand((N, K), generator=g, device="cuda") * 4 - 2).to(torch.bfloat16), "E2M1", "lut")
    # Uniform(-2, 2) operands give sums of 7168 products of magnitude ~100, where an absolute tolerance of 1e-2 is below
    # half a bf16 ulp.  The weight scales are lowered by 2^-7 (an exact shift of every product and every partial sum)
    # so that the outputs are of order one, the magnitude for which rtol 1e-2 / atol 1e-2 is stated.
    w_s -= 7
    cnt = torch.from_numpy(counts).cuda()
    c = ops.mx_gmm(a, a_s, w, w_s, cnt, K, "E2M1", "bf16")
    off = np.concatenate([[0], np.cumsum(counts)])
    rng = np.random.default_rng(2)
    for e in [int(np.argmax(counts)), int(np.argmin(np.where(counts > 0, counts, 1 << 30))), 7, 19]:
        if counts[e] == 0:
            continue
        pick = np.unique(np.concatenate([[0, counts[e] - 1], rng.integers(0, counts[e], 14)])) + off[e]
        gold = O.mx_gmm_f32(O.unpack_fp4(_np(a[pick])), _np(a_s[pick]), O.unpack_fp4(_np(w[e:e + 1])), _np(w_s[e:e + 1]), [len(pick)],
                            "E2M1", "E2M1")
        assert 0.2 < np.abs(gold).mean() < 5.0
        bad, worst = close_bf16(host(c[pick]), gold, rtol=1e-2, atol=1e-2)
        assert bad == 0, (e, bad, worst)
    c2 = ops.mx_gmm(a, a_s + 1, w, w_s, cnt, K, "E2M1", "bf16")
    assert torch.equal(c2.float(), c.float() * 2)
    del c2
    # group-order equivariance on every row: the same rows as groups in reverse expert order (every row lands in
    # another tile, next to other rows, under another group's position in the schedule) give the same row results
    order = list(range(E - 1, -1, -1))
    src = torch.cat([torch.arange(off[e], off[e + 1], device="cuda") for e in order])
    c_r = ops.mx_gmm(a[src].contiguous(), a_s[src].contiguous(), w[order].contiguous(), w_s[order].contiguous(),
                     torch.from_numpy(counts[order].copy()).cuda(), K, "E2M1", "bf16")
    assert torch.equal(c_r, c[src])


def test_config4_ffn_full_size():
    from catccos_amd import ops
    T, E, TOPK, K, N = 8192, 256, 8, 7168, 4096
    idx_h, p_h = W.softmax_topk_routing(T, E, TOPK, 41)
    idx, p = torch.from_numpy(idx_h.astype(np.int32)).cuda(), torch.from_numpy(p_h.astype(np.float32)).cuda()
    g = torch.Generator(device="cuda")
    g.manual_seed(42)
    x = torch.randn((T, K), generator=g, device="cuda").to(torch.bfloat16)
    w1 = torch.empty((E, N, K), dtype=torch.uint8, device="cuda")
    w1s = torch.empty((E, N, K // 32), dtype=torch.uint8, device="cuda")
    w2 = torch.empty((E, K, N // 2), dtype=torch.uint8, device="cuda")
    w2s = torch.empty((E, K, N // 64), dtype=torch.uint8, device="cuda")
    for e in range(E):
        w1[e], w1s[e] = _gpu_mx((N, K), 1000 + e, std=0.02, mode="lut")
        w2[e], w2s[e] = _gpu_mx((K, N // 2), 2000 + e, std=0.02, mode="lut")
    ws = torch.full((ops.ffn_workspace_bytes(T, K, N, E, TOPK),), 0xA5, dtype=torch.uint8, device="cuda")
    out = ops.dispatch_ffn_combine(x, idx, p, w1, w1s, w2, w2s, workspace=ws)
    # sampled tokens against the oracle chain restricted to their own experts (re-labelled 0..n-1)
    toks = np.array([0, 4097, 8191])
    used = np.unique(idx_h[toks])
    relabel = {int(e): i for i, e in enumerate(used)}
    sub_idx = np.vectorize(relabel.get)(idx_h[toks]).astype(np.int32)
    used_t = torch.from_numpy(used).cuda()
    gold = O.bf16_bits_to_f32(O.moe_ffn(host(x[toks]), sub_idx, p_h[toks].astype(np.float32), _np(w1[used_t]), _np(w1s[used_t]),
                                        _np(w2[used_t]), _np(w2s[used_t])))
    got = O.bf16_bits_to_f32(host(out[toks]))
    diff = np.abs(got - gold)
    assert (diff > 1e-2 + 1e-2 * np.abs(gold)).sum() <= got.size // 500 and diff.max() <= 5e-2, (diff.max(),)
    # ---- stage by stage at full size, on the kernel's own intermediates -------------------------------------
    lay = ops.ffn_workspace_layout(T, K, N, E, TOPK)
    rows = T * TOPK
    half = N // 2
    view = lambda name, nbytes: ws[lay[name]:lay[name] + nbytes]
    src2 = view("src2sorted", rows * 4).view(torch.int32)
    cnts = _np(view("counts", E * 4).view(torch.int32))
    assert np.array_equal(cnts, np.bincount(idx_h.reshape(-1), minlength=E))
    a_codes = view("a_codes", rows * K).view(rows, K)
    a_scales = view("a_scales", rows * lay["a_scales_pitch"]).view(rows, lay["a_scales_pitch"])[:, :K // 32]
    act_codes = view("act_codes", rows * half).view(rows, half)
    act_scales = view("act_scales", rows * (half // 32)).view(rows, half // 32)
    y = view("y", rows * K * 2).view(torch.int16).view(rows, K)
    # (1) dispatch: the eight destination rows of 64 sampled tokens hold the oracle's MX row of that token
    rng = np.random.default_rng(7)
    toks64 = np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 70)]))[:64]
    xq, xs = O.mx_quant_bf16(host(x[toks64]), "E4M3", "rne")
    dst = _np(src2.view(T, TOPK)[torch.from_numpy(toks64).cuda()])
    for j, t in enumerate(toks64):
        rows_t = torch.from_numpy(dst[j].astype(np.int64)).cuda()
        assert np.array_equal(_np(a_codes[rows_t]), np.repeat(xq[j:j + 1], TOPK, axis=0)), t
        assert np.array_equal(_np(a_scales[rows_t]), np.repeat(xs[j:j + 1], TOPK, axis=0)), t
    # (2) GMM1 + SwiGLU + requant and (3) GMM2 on 8 rows of each of 8 experts (first, last, six random rows)
    off4 = np.concatenate([[0], np.cumsum(cnts)])
    for e in [0, 17, 101, 128, 200, 255, int(np.argmax(cnts)), int(np.argmin(cnts))]:
        if cnts[e] == 0:
            continue
        pick = np.unique(np.concatenate([[0, cnts[e] - 1], rng.integers(0, cnts[e], 6)])) + off4[e]
        pk = torch.from_numpy(pick).cuda()
        _, _, gq, gs = O.gmm1_swiglu_quant(_np(a_codes[pk]), _np(a_scales[pk]), _np(w1[e:e + 1]), _np(w1s[e:e + 1]), [len(pick)])
        qa, sa = _np(act_codes[pk]), _np(act_scales[pk])
        deq, deq_g = O.mx_dequant(qa, sa), O.mx_dequant(gq, gs)
        bound = 0.13 * np.abs(deq_g) + 2.0 ** -5 * np.abs(deq_g).max(axis=1, keepdims=True) + 1e-9
        assert np.all(np.abs(deq - deq_g) <= bound), e
        bad, worst = close_bf16(host(y[pk]), O.mx_gmm_f32(qa, sa, _np(w2[e:e + 1]), _np(w2s[e:e + 1]), [len(pick)]))   # GMM2, strict, on the kernel's codes
        assert bad == 0, (e, bad, worst)
    # (2b) every one of the 65 536 rows: the instantiation that also writes the bf16 SwiGLU values, run on the chain's own
    # dispatched rows, gives the chain's codes and scales, and these are what the HIP quantizer (bit-exact against the
    # oracle elsewhere) and, on 8192 rows, the numpy oracle make of those bf16 values
    cnt_d = view("counts", E * 4).view(torch.int32)
    a_scales_p = view("a_scales", rows * lay["a_scales_pitch"]).view(rows, lay["a_scales_pitch"])
    codes_b, scales_b, act_b = ops.mx_gmm_swiglu_quant(a_codes, a_scales_p, w1, w1s, cnt_d, K, want_bf16=True)
    assert torch.equal(codes_b, act_codes) and torch.equal(scales_b, act_scales)
    hq, hs = ops.mx_quant(act_b, "E4M3", "rne")
    assert torch.equal(hq, act_codes) and torch.equal(hs, act_scales)
    for r0 in range(0, rows, 8 * 8192):
        oq, osc = O.mx_quant_bf16(host(act_b[r0:r0 + 8192]), "E4M3", "rne")
        assert np.array_equal(oq, _np(act_codes[r0:r0 + 8192])) and np.array_equal(osc, _np(act_scales[r0:r0 + 8192])), r0
    del codes_b, scales_b, hq, hs
    # (2c) rows permuted within every expert (each row in another 32-row block of another m-tile, the ragged tail tile
    # holding other rows): the bf16 SwiGLU values and the GMM2 outputs follow their rows
    gperm = torch.Generator(device="cuda")
    gperm.manual_seed(9)
    keys = torch.repeat_interleave(torch.arange(E, device="cuda"), cnt_d.long()).double() + torch.rand(rows, generator=gperm, device="cuda", dtype=torch.float64) * 0.5
    perm = torch.argsort(keys)
    codes_p, scales_p, act_p = ops.mx_gmm_swiglu_quant(a_codes[perm].contiguous(), a_scales_p[perm].contiguous(), w1, w1s, cnt_d, K, want_bf16=True)
    _assert_rows_follow(act_p.view(torch.int16), act_b.view(torch.int16)[perm], "gmm1 act")
    del act_b, act_p, codes_p, scales_p
    y_p = ops.mx_gmm(act_codes[perm].contiguous(), act_scales[perm].contiguous(), w2, w2s, cnt_d, half, "E4M3", "bf16")
    _assert_rows_follow(y_p.view(torch.int16), y[perm], "gmm2 y")
    del y_p
    # (4) combine: bit-exact on the 64 sampled tokens, from the kernel's own y rows
    y_rows = host(y[torch.from_numpy(dst.reshape(-1).astype(np.int64)).cuda()])
    local = np.arange(64 * TOPK, dtype=np.int32)
    assert np.array_equal(host(out[torch.from_numpy(toks64).cuda()]), O.unpermute_combine(y_rows, local, p_h[toks64].astype(np.float32)))
    # routing tables at full size: a permutation, keys non-decreasing, stable within a key
    s2s = ws[lay["sorted2src"]:lay["sorted2src"] + rows * 4].view(torch.int32)
    keys = idx.reshape(-1)[s2s.long()]
    assert torch.equal(torch.sort(s2s).values, torch.arange(rows, device="cuda", dtype=torch.int32))
    assert bool((keys[1:] >= keys[:-1]).all())
    same = keys[1:] == keys[:-1]
    assert bool((s2s[1:][same] > s2s[:-1][same]).all())
    assert torch.equal(src2[s2s.long()], torch.arange(rows, device="cuda", dtype=torch.int32))
    # doubling every gate weight doubles the bf16 output exactly (the combine multiplies, then adds in fp32)
    out2 = ops.dispatch_ffn_combine(x, idx, p * 2, w1, w1s, w2, w2s, workspace=ws)
    assert torch.equal(out2.float(), out.float() * 2)
    # (5) the same chain on pre-tiled weights (the weights-to-registers kernel in both matmuls): same bits at every stage
    w1t, w2t = ops.pretile_weights(w1, True), ops.pretile_weights(w2, False)
    keep_codes, keep_scales, keep_y = act_codes.clone(), act_scales.clone(), y.clone()
    ws.fill_(0x5A)
    out_t = ops.dispatch_ffn_combine(x, idx, p, w1t, w1s, w2t, w2s, workspace=ws)
    assert torch.equal(act_codes, keep_codes) and torch.equal(act_scales, keep_scales)
    assert torch.equal(y, keep_y) and torch.equal(out_t, out)
