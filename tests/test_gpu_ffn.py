"""The full single-device MoE FFN against the oracle chain."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W
from tests.gpu_util import dev, host, bf16_dev, close_bf16

pytestmark = pytest.mark.gpu


def _make(tokens, k, n, experts, top_k, seed):
    rng = np.random.default_rng(seed)
    x = W.normal_bf16((tokens, k), seed)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, seed + 1)
    w1 = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut") for _ in range(experts)]
    w2 = [O.mx_quant(O.bf16_round(rng.standard_normal((k, n // 2)).astype(np.float32) / np.sqrt(n // 2)), "E4M3", "lut") for _ in range(experts)]
    w1q, w1s = np.stack([a for a, _ in w1]), np.stack([b for _, b in w1])
    w2q, w2s = np.stack([a for a, _ in w2]), np.stack([b for _, b in w2])
    return x, idx, p, w1q, w1s, w2q, w2s


@pytest.mark.parametrize("tokens,k,n,experts,top_k", [(4, 256, 512, 4, 2), (64, 512, 1024, 16, 6), (300, 256, 512, 8, 8),
                                                      (512, 512, 512, 32, 4)])
def test_ffn_vs_oracle(tokens, k, n, experts, top_k):
    from catccos_amd import ops
    x, idx, p, w1q, w1s, w2q, w2s = _make(tokens, k, n, experts, top_k, seed=tokens)
    ws_bytes = ops.ffn_workspace_bytes(tokens, k, n, experts, top_k)
    workspace = torch.full((ws_bytes,), 0xA5, dtype=torch.uint8, device="cuda")      # poisoned, as the reference's regression mode
    out = ops.dispatch_ffn_combine(bf16_dev(x), dev(idx), dev(p), dev(w1q), dev(w1s), dev(w2q), dev(w2s), workspace=workspace)
    gold, st = O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s, stages=True)
    got = host(out)
    # End to end the chain holds two requantisations whose rounding decisions can flip on a
    # one-ulp difference of the bf16 GMM1 output, so single elements may move by more than a
    # matmul's tolerance: require 99.9% within rtol/atol 1e-2, none beyond 5e-2, and the
    # reference's mean-bias bound; the matmul stages are checked one by one below.
    gold_f = O.bf16_bits_to_f32(gold)
    bad, worst = close_bf16(got, gold_f)
    assert bad <= got.size // 1000 and worst <= 5e-2, (bad, worst)
    ok, err, eb = O.verify_bf16(got, gold_f, 1 << 20)
    assert eb <= 2.0 ** -7 and err <= got.size // 1000, (err, eb)
    # integer stages are bit-exact: routing tables and the dispatched MX rows
    lay = ops.ffn_workspace_layout(tokens, k, n, experts, top_k)
    rows = tokens * top_k
    w = workspace.cpu().numpy()
    assert np.array_equal(w[lay["src2sorted"]:lay["src2sorted"] + rows * 4].view(np.int32), st["src2sorted"])
    assert np.array_equal(w[lay["sorted2src"]:lay["sorted2src"] + rows * 4].view(np.int32), st["sorted2src"])
    assert np.array_equal(w[lay["counts"]:lay["counts"] + experts * 4].view(np.int32), st["counts"])
    assert np.array_equal(w[lay["a_codes"]:lay["a_codes"] + rows * k].reshape(rows, k), st["aq"])
    pitch = lay["a_scales_pitch"]                     # scale rows sit at a pitch of whole 128-byte lines
    assert np.array_equal(w[lay["a_scales"]:lay["a_scales"] + rows * pitch].reshape(rows, pitch)[:, :k // 32], st["asc"])
    # stage by stage on the kernel's own intermediates
    half = n // 2
    qa = w[lay["act_codes"]:lay["act_codes"] + rows * half].reshape(rows, half)
    sa = w[lay["act_scales"]:lay["act_scales"] + rows * (half // 32)].reshape(rows, half // 32)
    deq, deq_g = O.mx_dequant(qa, sa), O.mx_dequant(st["qa"], st["sa"])
    bound = 0.13 * np.abs(deq_g) + 2.0 ** -5 * np.abs(deq_g).max(axis=1, keepdims=True)
    assert np.all(np.abs(deq - deq_g) <= bound)
    y = w[lay["y"]:lay["y"] + rows * k * 2].view(np.uint16).reshape(rows, k)
    bad, worst = close_bf16(y, O.mx_gmm_f32(qa, sa, w2q, w2s, st["counts"]))          # GMM2 on the same codes
    assert bad == 0, (bad, worst)
    assert np.array_equal(got, O.unpermute_combine(y, st["src2sorted"], p))            # combine is bit-exact
    # second launch on the same (now dirty) workspace gives the same bits
    out2 = ops.dispatch_ffn_combine(bf16_dev(x), dev(idx), dev(p), dev(w1q), dev(w1s), dev(w2q), dev(w2s), workspace=workspace)
    assert torch.equal(out, out2)


def test_several_shapes_on_one_dirty_workspace():
    """The reference's case-list mode runs several shapes in one process on one workspace that was poisoned once
    (examples/ascend950_dispatch_ffn_combine/main.cpp:150-170, 217-252): a large shape first, then smaller ones on
    what it left behind, then the large one again.  Every result must equal that of a run on a fresh workspace."""
    from catccos_amd import ops
    shapes = [(512, 512, 1024, 32, 4), (4, 256, 512, 4, 2), (300, 256, 512, 8, 8), (64, 512, 1024, 16, 6), (512, 512, 1024, 32, 4)]
    big = max(ops.ffn_workspace_bytes(*s) for s in shapes)
    shared = torch.full((big,), 0xA5, dtype=torch.uint8, device="cuda")
    for i, (tokens, k, n, experts, top_k) in enumerate(shapes):
        x, idx, p, w1q, w1s, w2q, w2s = _make(tokens, k, n, experts, top_k, seed=tokens + 11)
        args = (bf16_dev(x), dev(idx), dev(p), dev(w1q), dev(w1s), dev(w2q), dev(w2s))
        fresh = torch.zeros(ops.ffn_workspace_bytes(tokens, k, n, experts, top_k), dtype=torch.uint8, device="cuda")
        want = ops.dispatch_ffn_combine(*args, workspace=fresh)
        got = ops.dispatch_ffn_combine(*args, workspace=shared)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (i, tokens)
        if tokens <= 64:                                    # and against the oracle chain
            gold = O.bf16_bits_to_f32(O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s))
            bad, worst = close_bf16(host(got), gold)
            assert bad <= got.numel() // 1000 and worst <= 5e-2, (bad, worst)


def test_ffn_rejects_top_k_beyond_the_combine_limit_before_any_launch():
    from catccos_amd import _lib
    lib = _lib.load()
    z = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    out = torch.full((1 << 16,), 0x5A, dtype=torch.uint8, device="cuda")
    ws = torch.full((1 << 22,), 0xA5, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    rc = lib.catccos_ascend950_dispatch_ffn_combine(0, None, 0, p, p, p, p, p, p, p, out.data_ptr(), ws.data_ptr(), None,
                                                    2, 256, 512, 128, 65, 1)
    torch.cuda.synchronize()
    assert rc == -1 and b"64" in lib.cmx_last_error()
    assert bool((ws == 0xA5).all()) and bool((out == 0x5A).all())          # nothing was launched


def test_workspace_size_matches_reference_formula():
    from catccos_amd import ops
    for (m, k, n, e, t) in [(4, 7168, 4096, 16, 6), (512, 7168, 4096, 16, 6), (8192, 7168, 4096, 256, 8), (256, 7168, 1024, 16, 6)]:
        assert ops.ffn_workspace_bytes(m, k, n, e, t) == O.ffn_workspace_bytes(m, k, n, 1, 1, e, t)
        assert ops.ffn_workspace_layout(m, k, n, e, t)["y"] + m * t * k * 2 <= ops.ffn_workspace_bytes(m, k, n, e, t)


def test_ffn_rejects_bad_shapes():
    from catccos_amd import _lib
    lib = _lib.load()
    z = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    args = lambda m, k, n, e, t, r: (0, None, 0, p, p, p, p, p, p, p, p, p, None, m, k, n, e, t, r)
    assert lib.catccos_ascend950_dispatch_ffn_combine(*args(4, 128, 512, 4, 2, 1)) == -1     # K % 256
    assert lib.catccos_ascend950_dispatch_ffn_combine(*args(4, 256, 256, 4, 2, 1)) == -1     # N % 512
    assert lib.catccos_ascend950_dispatch_ffn_combine(*args(4, 256, 512, 4, 5, 1)) == -1     # topK > experts
    assert lib.catccos_ascend950_dispatch_ffn_combine(*args(4, 256, 512, 4, 2, 2)) == -1     # rankSize


def test_ffn_chain_replays_from_a_hip_graph():
    """The chain makes no allocation, no memset and no host synchronisation, so it can be captured into a HIP
    graph once and replayed: three replays, each after the program changed the tokens in place and did eager work
    of its own, every one compared bit for bit with an eager run on the same inputs."""
    from catccos_amd import ops
    tokens, k, n, experts, top_k = 96, 512, 512, 8, 4
    x, idx, p, w1q, w1s, w2q, w2s = _make(tokens, k, n, experts, top_k, seed=77)
    xd, idxd, pd = bf16_dev(x), dev(idx), dev(p)
    w1d, w1sd, w2d, w2sd = dev(w1q), dev(w1s), dev(w2q), dev(w2s)
    ws = torch.empty(ops.ffn_workspace_bytes(tokens, k, n, experts, top_k), dtype=torch.uint8, device="cuda")
    ws_eager = torch.empty_like(ws)
    out = torch.zeros((tokens, k), dtype=torch.bfloat16, device="cuda")
    run = lambda o, w: ops.dispatch_ffn_combine(xd, idxd, pd, w1d, w1sd, w2d, w2sd, workspace=w, out=o)
    run(out, ws)                                   # first launches set kernel attributes: outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            run(out, ws)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        xd.copy_(bf16_dev(W.normal_bf16((tokens, k), 100 + rep)))       # new tokens in the captured buffer
        expect = torch.zeros_like(out)
        run(expect, ws_eager)                      # eager work between the replays
        torch.cuda.synchronize()
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), expect.view(torch.int16)), rep


def test_capture_right_after_init():
    """A process whose first launches of the library's kernels happen inside a stream capture, after cmx_init() alone
    (tests/capture_after_init_child.py): the FFN chain and the allocation-free grouped matmul replay bit for bit."""
    import os
    import subprocess
    import sys
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "capture_after_init_child.py")
    r = subprocess.run([sys.executable, child], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "CAPTURE-OK" in r.stdout, (r.returncode, r.stdout[-2000:], r.stderr[-2000:])
