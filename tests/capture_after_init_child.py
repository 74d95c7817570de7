"""Child process of test_gpu_ffn.test_capture_right_after_init: in a process that has launched none of the library's
kernels, cmx_init() alone must be enough to capture the FFN chain (on row-major and on pre-tiled weights) and the
allocation-free grouped matmul into a HIP graph (no kernel's first launch may need set-up that a capture forbids; the
one-off weight tiling pass runs before the capture, as it would at weight-load time).  The graph is replayed twice, with eager
work in between, and every replay compared bit for bit with eager runs made afterwards.  Prints CAPTURE-OK."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from catccos_amd import ops                     # noqa: E402
from catccos_amd import workloads as W          # noqa: E402
from oracle import mx_oracle as O               # noqa: E402
from tests.gpu_util import dev, bf16_dev        # noqa: E402


def main() -> int:
    tokens, k, n, experts, top_k = 96, 512, 1024, 8, 4
    rng = np.random.default_rng(5)
    x = W.normal_bf16((tokens, k), 5)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, 6)
    w1 = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut") for _ in range(experts)]
    w2 = [O.mx_quant(O.bf16_round(rng.standard_normal((k, n // 2)).astype(np.float32) / np.sqrt(n // 2)), "E4M3", "lut") for _ in range(experts)]
    w1d, w1sd = dev(np.stack([a for a, _ in w1])), dev(np.stack([b for _, b in w1]))
    w2d, w2sd = dev(np.stack([a for a, _ in w2])), dev(np.stack([b for _, b in w2]))
    xd, idxd, pd = bf16_dev(x), dev(idx), dev(p)
    # operands of the allocation-free grouped matmul: rows already sorted by expert
    counts_h = np.array([20, 0, 257, 5, 40, 0, 60, 2], dtype=np.int32)
    m = int(counts_h.sum())
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    aqd, ascd, cnt = dev(aq), dev(asc), dev(counts_h)
    ws = torch.empty(ops.ffn_workspace_bytes(tokens, k, n, experts, top_k), dtype=torch.uint8, device="cuda")
    ws_eager = torch.empty_like(ws)
    out = torch.zeros((tokens, k), dtype=torch.bfloat16, device="cuda")
    out_t = torch.zeros((tokens, k), dtype=torch.bfloat16, device="cuda")
    ws_t = torch.empty_like(ws)
    codes = torch.zeros((m, n // 2), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((m, ops.scale_cols(n // 2)), dtype=torch.uint8, device="cuda")

    def run(o, w, c, s):
        ops.dispatch_ffn_combine(xd, idxd, pd, w1d, w1sd, w2d, w2sd, workspace=w, out=o)
        ops.mx_gmm_swiglu_quant_noalloc(aqd, ascd, w1d, w1sd, cnt, k, c, s, None)

    ops.init()                                   # the only library call before the capture, apart from the tiling pass
    w1t, w2t = ops.pretile_weights(w1d, True), ops.pretile_weights(w2d, False)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            run(out, ws, codes, scales)
            ops.dispatch_ffn_combine(xd, idxd, pd, w1t, w1sd, w2t, w2sd, workspace=ws_t, out=out_t)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(2):
        xd.copy_(bf16_dev(W.normal_bf16((tokens, k), 200 + rep)))
        out.fill_(7.0)
        out_t.fill_(7.0)
        codes.fill_(0xEE)
        scales.fill_(0xEE)
        graph.replay()
        torch.cuda.synchronize()
        e_out, e_codes, e_scales = torch.zeros_like(out), torch.zeros_like(codes), torch.zeros_like(scales)
        run(e_out, ws_eager, e_codes, e_scales)          # eager, after the replay (and between the replays)
        torch.cuda.synchronize()
        if not (torch.equal(out.view(torch.int16), e_out.view(torch.int16)) and torch.equal(codes, e_codes) and torch.equal(scales, e_scales)
                and torch.equal(out_t.view(torch.int16), e_out.view(torch.int16))):
            print(f"replay {rep} differs from the eager run", flush=True)
            return 1
    print("CAPTURE-OK", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
