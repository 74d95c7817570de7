#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ by running the reference's own Python goldens.

Run once, in the build container, where the reference checkout is present:

    python tests/golden/make_fixtures.py [/root/reference]

Only the vectors (inputs and expected outputs, as .npz) are committed; nothing of the reference travels.
What is imported, and why each needs the real thing rather than a restatement:

* ``examples/utils/gen_mx_quant_allgather_data.py`` -- ``_quantize_fp8`` (both GEN_DATA_QUANT_BACKENDs),
  ``_quantize`` / ``_quantize_to_fp4_lut`` / ``_pack_fp4_nibbles``: the quantizer goldens, on a small matrix
  that holds every rounding tie, signed zeros, all-zero and tiny blocks, outliers and non-finite values.
* ``examples/utils/gen_data_moe.py`` -- ``generate_dispatch_ffn_combine_mx`` on a tiny shape: the composition of
  the FFN chain (which half of GMM1 gets the SiLU, where the bf16 roundings sit, which quantizer rounding each
  operand gets, how the combine accumulates).

* ``examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/gen_data_mxfp8_mmrs.py`` -- ``gen_data`` on a tiny shape, B
  stored both ways: the operand and scale FILE layouts of the dense MXFP8 example ([K, N] codes with [K/64, N, 2]
  scales, and the transposed pair), its per-element E5M2 table quantizer and its ``golden`` / ``golden_low`` pair.
* ``examples/utils/gen_data_fp4_mx_alltoallv_gmm.py`` -- ``generate_data`` on a tiny shape: the legacy
  ``MXFP4MatrixQuantizer`` (E2M1 table rounding, bit-level nibble packing), the file layouts of the FP4 grouped-matmul
  example and its fp32 golden.

``gen_data_dispatch_gmm_dequant_swiglu.py`` is not imported (it needs an NPU-only package and deletes
``./output`` at import time).
"""
from __future__ import annotations

import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def _u8(t):
    import torch
    return t.contiguous().view(torch.uint8).numpy().copy()


def quant_input() -> np.ndarray:
    """fp32 [12, 128] (values exactly representable in bf16): four 32-blocks per row."""
    rng = np.random.default_rng(20240601)
    x = rng.standard_normal((12, 128)).astype(np.float32)
    x[1] *= 37.0
    x[2] *= 2.0 ** -9
    x[3, :32] = 0.0                                    # all-zero block
    x[3, 32:64] = 1e-13                                # below the golden's epsilon
    x[3, 64:96] = np.float32(2.0 ** -126)              # smallest normal
    # every E4M3 midpoint between neighbours in [1, 2): block maximum 448 -> exponent 0, so they are ties as stored
    x[4, 0] = 448.0
    x[4, 1:9] = [1.0625, 1.1875, 1.3125, 1.4375, 1.5625, 1.6875, 1.8125, 1.9375]
    x[4, 9:17] = [-1.0625, -1.1875, -1.3125, -1.4375, -1.5625, -1.6875, -1.8125, -1.9375]
    x[4, 17:21] = [2.0 ** -10, -(2.0 ** -10), 3 * 2.0 ** -10, -(2.0 ** -11)]      # subnormal ties and underflow
    x[4, 21:25] = [0.0, -0.0, 2.0 ** -12, -(2.0 ** -12)]
    x[4, 25:32] = 0.0
    # every E2M1 midpoint, block maximum 6 -> exponent 0
    x[5, 0] = 6.0
    x[5, 1:8] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0]
    x[5, 8:15] = [-0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0]
    x[5, 15:32] = 0.0
    # every E1M2 midpoint, block maximum 1.75 -> exponent 0
    x[6, 0] = 1.75
    x[6, 1:8] = [0.125, 0.375, 0.625, 0.875, 1.125, 1.375, 1.625]
    x[6, 8:15] = [-0.125, -0.375, -0.625, -0.875, -1.125, -1.375, -1.625]
    x[6, 15:32] = 0.0
    x[7, 5] = 511.0                                    # clips to 448 after scaling by the block exponent
    x[7, 40] = -7.9
    x[8] *= 100.0
    # round everything to bf16 (the device quantizer's input type); done before the non-finite entries go in
    b = x.view(np.uint32)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16 << 16).astype(np.uint32)
    x = b.view(np.float32).copy()
    x[9, 3] = np.inf                                   # non-finite blocks: one Inf, one -Inf, one NaN, one mixed
    x[9, 40] = -np.inf
    x[9, 70] = np.nan
    x[9, 100] = np.nan
    x[9, 101] = np.inf
    return x


def main() -> int:
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    utils = os.path.join(ref, "examples", "utils")
    if not os.path.isdir(utils):
        print(f"reference checkout not found at {ref}: fixtures are made in the build container only", file=sys.stderr)
        return 2
    sys.path.insert(0, utils)
    import torch
    import gen_mx_quant_allgather_data as Q                         # noqa: E402  (reference module)

    out = {}
    x = quant_input()
    out["x"] = x
    xt = torch.from_numpy(x)
    finite_rows = 9                                                 # rows 0..8 hold finite values only
    for backend in ("lut", "native"):
        Q._QUANT_BACKEND = backend
        for fmt in ("E4M3", "E5M2"):
            q, s, d = Q._quantize_fp8(xt[:finite_rows].clone(), fmt, axis=1)
            out[f"fp8_{fmt}_{backend}_codes"] = _u8(q)
            out[f"fp8_{fmt}_{backend}_scales"] = _u8(s.to(torch.float8_e8m0fnu))
            out[f"fp8_{fmt}_{backend}_dequant"] = d.numpy().copy()
        # a row count that is not a multiple of 32 along the quantised axis and an odd block count (scale padding)
        q, s, _ = Q._quantize_fp8(xt[:finite_rows, :96].clone(), "E4M3", axis=1)
        out[f"fp8_E4M3_{backend}_n96_codes"] = _u8(q)
        out[f"fp8_E4M3_{backend}_n96_scales"] = _u8(s.to(torch.float8_e8m0fnu))
    # non-finite inputs (row 9): what the golden does with them, for every format and backend
    for backend in ("lut", "native"):
        Q._QUANT_BACKEND = backend
        for fmt in ("E4M3", "E5M2"):
            q, s, _ = Q._quantize_fp8(xt[9:10].clone(), fmt, axis=1)
            out[f"fp8_{fmt}_{backend}_nonfinite_codes"] = _u8(q)
            out[f"fp8_{fmt}_{backend}_nonfinite_scales"] = _u8(s.to(torch.float8_e8m0fnu))
    Q._QUANT_BACKEND = "lut"
    for fmt in ("E2M1", "E1M2"):
        qv, s, d = Q._quantize(xt[:finite_rows].clone(), fmt, axis=1)
        out[f"fp4_{fmt}_values"] = qv.numpy().copy()
        out[f"fp4_{fmt}_scales"] = _u8(s.to(torch.float8_e8m0fnu))
        # codes the way the FP4 example packs them: indices of the scaled values in the 16-entry table
        sc = s[:, : x.shape[1] // 32].repeat_interleave(32, dim=1)
        _, idx = Q._quantize_to_fp4_lut(xt[:finite_rows] / sc, fmt)
        out[f"fp4_{fmt}_codes"] = idx.numpy().copy()
        out[f"fp4_{fmt}_packed"] = Q._pack_fp4_nibbles(idx).numpy().copy()
        _, s9, _ = Q._quantize(xt[9:10].clone(), fmt, axis=1)
        out[f"fp4_{fmt}_nonfinite_scales"] = _u8(s9.to(torch.float8_e8m0fnu))
        sc9 = s9[:, : x.shape[1] // 32].repeat_interleave(32, dim=1)
        _, idx9 = Q._quantize_to_fp4_lut(xt[9:10] / sc9, fmt)
        out[f"fp4_{fmt}_nonfinite_codes"] = idx9.numpy().copy()
    np.savez_compressed(os.path.join(HERE, "quant_vectors.npz"), **out)
    print("wrote quant_vectors.npz:", ", ".join(sorted(out)))

    # ---- the FFN chain on a tiny shape ----------------------------------------------------------------------
    import gen_data_moe as G                                        # noqa: E402  (reference module)
    m, k, n, top_k, experts = 5, 256, 512, 2, 3
    with tempfile.TemporaryDirectory() as tmp:
        G.generate_dispatch_ffn_combine_mx(
            m, k, n, top_k, active_num=m * top_k, capacity=m * top_k, drop_pad_mode=0, ep=1, expert_per_rank=experts,
            batch_size=1, max_output_size=m * top_k, dtype=torch.bfloat16, data_path=tmp, routing_mode="random")

        def rd(name, dtype, shape):
            return np.fromfile(os.path.join(tmp, name), dtype=dtype).reshape(shape)
        ffn = dict(
            shape=np.array([m, k, n, top_k, experts], dtype=np.int64),
            x=rd("in_routing_matrix_a_0.bin", np.uint16, (m, k)),
            expert_idx=rd("in_routing_expert_idx_0.bin", np.int32, (m, top_k)),
            gate_weight=rd("in_gather_gate_weight_0.bin", np.float32, (m, top_k)),
            w1=rd("in_gmm_matrix_b_0.bin", np.uint8, (experts, n, k)),
            w1_scale=rd("in_gmm_matrix_b_scale_0.bin", np.uint8, (experts, n, k // 32)),
            w2=rd("in_gmm_matrix_b2_0.bin", np.uint8, (experts, k, n // 2)),
            w2_scale=rd("in_gmm_matrix_b2_scale_0.bin", np.uint8, (experts, k, n // 64)),
            sorted2src=rd("in_gather_expanded_row_idx_0.bin", np.int32, (m * top_k,)),
            y=rd("in_gather_permuted_0.bin", np.uint16, (m * top_k, k)),
            out=rd("out_gather_combine_0.bin", np.uint16, (m, k)),
        )
    np.savez_compressed(os.path.join(HERE, "ffn_tiny.npz"), **ffn)
    print("wrote ffn_tiny.npz:", ", ".join(f"{a}{tuple(v.shape)}" for a, v in ffn.items()))

    # ---- dense MXFP8 matmul example: file layouts and the double golden ------------------------------------------
    sys.path.insert(0, os.path.join(ref, "examples", "ascend950_mxfp8_matmul_reduce_scatter", "scripts"))
    import gen_data_mxfp8_mmrs as D                                 # noqa: E402  (reference module)
    m, k, n = 8, 128, 16
    mm = dict(shape=np.array([m, k, n], dtype=np.int64))
    torch.manual_seed(11)                                           # gen_data draws A [m, k], then B [k, n]
    mm["a_src"] = torch.randn((m, k), dtype=torch.float32).numpy().copy()
    mm["b_src"] = torch.randn((k, n), dtype=torch.float32).numpy().copy()
    for trans_b in (1, 0):                                          # 1 is what the example's run.sh passes
        torch.manual_seed(11)                                       # the same random matrices for both orientations
        with tempfile.TemporaryDirectory() as tmp:
            c_fp32, c_bf16 = D.gen_data(0, m, k, n, 0, trans_b, tmp)
            for what in ("a", "b", "a_scale", "b_scale"):
                mm[f"tb{trans_b}_{what}"] = np.fromfile(os.path.join(tmp, f"rank_0_{what}.bin"), dtype=np.uint8)
        mm[f"tb{trans_b}_golden"] = c_fp32.numpy().copy()
        mm[f"tb{trans_b}_golden_low"] = c_bf16.view(torch.uint16).numpy().copy()
    np.savez_compressed(os.path.join(HERE, "mmrs_tiny.npz"), **mm)
    print("wrote mmrs_tiny.npz:", ", ".join(f"{a}{tuple(v.shape)}" for a, v in mm.items()))

    # ---- FP4 grouped matmul example ---------------------------------------------------------------------------------
    import argparse
    import gen_data_fp4_mx_alltoallv_gmm as F                       # noqa: E402  (reference module)
    from utils import DataType                                      # noqa: E402  (reference module)
    m, k, n, experts = 24, 128, 32, 3
    torch.manual_seed(12)                                           # generate_data draws A [1, m, k], then B [1, E, k, n]
    a_src = F.random_uniform(-2.0, 2.0, size=(1, m, k)).numpy().copy()[0]
    b_src = F.random_uniform(-2.0, 2.0, size=(1, experts, k, n)).numpy().copy()[0]
    torch.manual_seed(12)
    with tempfile.TemporaryDirectory() as tmp:
        F.generate_data(argparse.Namespace(out_type=DataType.FLOAT16, rank_size=1, m=m, n=n, k=k, trans_a=0, trans_b=0,
                                           expert=experts, ep=1, data_dir=tmp))
        rd = lambda name, dtype: np.fromfile(os.path.join(tmp, name), dtype=dtype)
        f4 = dict(
            shape=np.array([m, k, n, experts], dtype=np.int64), a_src=a_src, b_src=b_src,
            input_a=rd("input_a_0.bin", np.uint8), input_a_scale=rd("input_a_scale_0.bin", np.uint8),
            input_b=rd("input_b_0.bin", np.uint8), input_b_scale=rd("input_b_scale_0.bin", np.uint8),
            local_tokens_per_expert=rd("local_tokens_per_expert_0.bin", np.int32),
            global_tokens_per_local_expert=rd("global_tokens_per_local_expert_0.bin", np.int32),
            golden=rd("golden_0.bin", np.float32).reshape(m, n),
        )
    np.savez_compressed(os.path.join(HERE, "fp4_gmm_tiny.npz"), **f4)
    print("wrote fp4_gmm_tiny.npz:", ", ".join(f"{a}{tuple(v.shape)}" for a, v in f4.items()))
    return 0


if __name__ == "__main__":
    sys.exit(main())
