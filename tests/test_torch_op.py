"""The torch.ops.catccos surface (reference: examples/torch_binding/src/torch_bindings.cpp:109-387)."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from catccos_amd import workloads as W


def test_schemas_registered_without_a_gpu():
    import catccos_amd.torch_op  # noqa: F401
    s = torch.ops.catccos.ascend950_dispatch_ffn_combine.default._schema
    assert [a.name for a in s.arguments] == ["x", "expert_idx", "gate_weight", "w1", "w1_scale", "w2", "w2_scale"]
    assert str(torch.ops.catccos.init.default._schema).startswith("catccos::init(int rank_id, int rank_size, int local_mem_size, str ip_port)")
    assert torch.ops.catccos.finalize() == 0                 # finalize before init is a no-op, as in the reference
    with pytest.raises(RuntimeError, match="invalid rank_id"):
        torch.ops.catccos.init(-1, 1, 1 << 20, "tcp://127.0.0.1:1")
    with pytest.raises(RuntimeError, match="ip_port is empty"):
        torch.ops.catccos.init(0, 1, 1 << 20, "")
    with pytest.raises(RuntimeError, match="rank_size must be 1"):
        torch.ops.catccos.init(0, 2, 1 << 20, "tcp://127.0.0.1:1")


@pytest.mark.gpu
def test_ffn_op_matches_oracle_and_checks_arguments():
    import catccos_amd.torch_op  # noqa: F401
    tokens, k, n, experts, top_k = 48, 256, 512, 4, 2
    rng = np.random.default_rng(9)
    x = W.normal_bf16((tokens, k), 9)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, 10)
    w1 = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut") for _ in range(experts)]
    w2 = [O.mx_quant(O.bf16_round(rng.standard_normal((k, n // 2)).astype(np.float32) / np.sqrt(n // 2)), "E4M3", "lut") for _ in range(experts)]
    w1q, w1s = np.stack([a for a, _ in w1]), np.stack([b for _, b in w1])
    w2q, w2s = np.stack([a for a, _ in w2]), np.stack([b for _, b in w2])
    dev = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).cuda().view(dt)
    xd = dev(x.view(np.int16), torch.bfloat16)
    args = [xd, dev(idx.astype(np.int32), torch.int32), dev(p.astype(np.float32), torch.float32),
            dev(w1q, torch.float8_e4m3fn), dev(w1s, torch.float8_e8m0fnu), dev(w2q, torch.float8_e4m3fn), dev(w2s, torch.float8_e8m0fnu)]
    with pytest.raises(RuntimeError, match="init"):
        torch.ops.catccos.ascend950_dispatch_ffn_combine(*args)
    assert torch.ops.catccos.init(0, 1, 1 << 30, "tcp://127.0.0.1:1") == 0
    assert torch.ops.catccos.init(0, 1, 1 << 30, "tcp://127.0.0.1:1") == 0          # idempotent
    try:
        y = torch.ops.catccos.ascend950_dispatch_ffn_combine(*args)
        y2 = torch.ops.catccos.ascend950_dispatch_ffn_combine(*args)                 # cached (now dirty) workspace
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (tokens, k) and torch.equal(y, y2)
        got = y.view(torch.int16).cpu().numpy().view(np.uint16)
        gold = O.bf16_bits_to_f32(O.moe_ffn(x, idx, p, w1q, w1s, w2q, w2s))
        diff = np.abs(O.bf16_bits_to_f32(got) - gold)
        assert (diff > 1e-2 + 1e-2 * np.abs(gold)).sum() <= got.size // 1000 and diff.max() <= 5e-2
        bad = list(args); bad[3] = args[3].view(torch.uint8)
        with pytest.raises(RuntimeError, match="w1 must have dtype"):
            torch.ops.catccos.ascend950_dispatch_ffn_combine(*bad)
        bad = list(args); bad[1] = args[1][:, :1]
        with pytest.raises(RuntimeError, match="contiguous|routing"):
            torch.ops.catccos.ascend950_dispatch_ffn_combine(*bad)
        bad = list(args); bad[0] = args[0][:, :128].contiguous()
        with pytest.raises(RuntimeError, match="divisible|shape"):
            torch.ops.catccos.ascend950_dispatch_ffn_combine(*bad)
    finally:
        assert torch.ops.catccos.finalize() == 0


@pytest.mark.gpu
def test_pretiled_ops_give_the_bits_of_the_reference_op():
    import catccos_amd.torch_op  # noqa: F401
    tokens, k, n, experts, top_k = 200, 512, 1024, 8, 4
    rng = np.random.default_rng(19)
    x = W.normal_bf16((tokens, k), 19)
    idx, p = W.softmax_topk_routing(tokens, experts, top_k, 20)
    w1 = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) / np.sqrt(k)), "E4M3", "lut") for _ in range(experts)]
    w2 = [O.mx_quant(O.bf16_round(rng.standard_normal((k, n // 2)).astype(np.float32) / np.sqrt(n // 2)), "E4M3", "lut") for _ in range(experts)]
    dev = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).cuda().view(dt)
    args = [dev(x.view(np.int16), torch.bfloat16), dev(idx.astype(np.int32), torch.int32), dev(p.astype(np.float32), torch.float32),
            dev(np.stack([a for a, _ in w1]), torch.float8_e4m3fn), dev(np.stack([b for _, b in w1]), torch.float8_e8m0fnu),
            dev(np.stack([a for a, _ in w2]), torch.float8_e4m3fn), dev(np.stack([b for _, b in w2]), torch.float8_e8m0fnu)]
    assert torch.ops.catccos.init(0, 1, 1 << 30, "tcp://127.0.0.1:1") == 0
    try:
        y = torch.ops.catccos.ascend950_dispatch_ffn_combine(*args)
        w1t, w2t = torch.ops.catccos.ascend950_pretile_ffn_weights(args[3], args[5])
        assert w1t.dtype == torch.uint8 and w1t.numel() == args[3].numel() and w2t.numel() == args[5].numel()
        yt = torch.ops.catccos.ascend950_dispatch_ffn_combine_pretiled(args[0], args[1], args[2], w1t, args[4], w2t, args[6])
        assert torch.equal(y, yt)
        with pytest.raises(RuntimeError, match="wrong size"):
            torch.ops.catccos.ascend950_dispatch_ffn_combine_pretiled(args[0], args[1], args[2], w1t[:-16], args[4], w2t, args[6])
        with pytest.raises(RuntimeError, match="must have dtype"):
            torch.ops.catccos.ascend950_dispatch_ffn_combine_pretiled(*args)       # row-major weights handed to the pre-tiled op
        with pytest.raises(RuntimeError, match="divisible by 512"):
            torch.ops.catccos.ascend950_pretile_ffn_weights(args[3][:, :, :256].contiguous(), args[5][:, :256].contiguous())
    finally:
        torch.ops.catccos.finalize()
