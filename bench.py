#!/usr/bin/env python3
"""Benchmark of the MI355X MX compute core (one GPU).

Headline step = one pass of the MoE grouped matmul with fused dequant + SwiGLU + MX requant
(the headline configuration, "config 3": E=16 local experts, 4096 tokens x top-8 Zipf-routed = 32768 ragged rows,
H=7168, W_gate/up [16, 4096, 7168] MXFP8) through the C ABI, inputs resident in HBM.
`value` = 2*rows*K*N flop / step time in TFLOP/s.  The same JSON line carries

  roofline      the grouped-matmul kernel against the dense MXFP8 MFMA peak (HIP-event timing on the
                launch stream), and in `extra` the quantizer / dense GEMM / FFN / FP4 / routing kernels
                each against its own bound;
  cpu_baseline  the numpy oracle of the same step timed on the host cores over a bounded sample.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME]] [--no-cpu]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MXFP8_PEAK_TFLOPS = 5000.0
MXFP4_PEAK_TFLOPS = 10100.0
INT8_PEAK_TOPS = 5000.0
SEED = 20240607


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed launches first; the launch time keeps falling for about 25 launches after an idle GPU")
    ap.add_argument("--only", type=str, default="", help="comma list of extras: quant,gemm,ffn,fp4,int8,routing,idle,copycal (default: all but copycal)")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(no collectives, no multi-device sharding in this tier)", file=sys.stderr)
        return 2

    import torch
    from catccos_amd import _lib, ops, workloads as W

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    lib = _lib.load()          # raises if the HIP library is missing: there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    K_STEPS, WARM = args.steps, args.warmup

    def hip_time(fn, steps=K_STEPS, warm=max(WARM, 25)):
        """Average duration (s) of fn() over `steps` launches, HIP events on the launch stream (the extras: at least 25
        untimed launches and 30 ms first, past the power-management ramp that follows a change of load)."""
        t_warm = time.perf_counter()
        while True:
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            if time.perf_counter() - t_warm >= 0.03:      # the clock needs about 20 ms of a new load to settle, however many launches that is
                break
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / steps

    def quant_weights(e, n, k, std, seed):
        """[e, n, k] MXFP8 weights: N(0, std) bf16 quantised per expert by the GPU quantizer (table rounding)."""
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        codes = torch.empty((e, n, k), dtype=torch.uint8, device=dev)
        scales = torch.empty((e, n, ops.scale_cols(k)), dtype=torch.uint8, device=dev)
        for i in range(e):
            w = (torch.randn((n, k), generator=g, device=dev) * std).to(torch.bfloat16)
            q, s = ops.mx_quant(w, "E4M3", "lut")
            codes[i], scales[i] = q, s
        return codes, scales

    # ------------------------------------------------------------------ headline: config 3 ----
    E, T, TOPK, H, N = 16, 4096, 8, 7168, 4096
    idx = W.zipf_routing(T, E, TOPK, SEED)
    counts_h = np.bincount(idx.reshape(-1), minlength=E).astype(np.int32)
    rows = int(counts_h.sum())
    counts = torch.from_numpy(counts_h).to(dev)
    g = torch.Generator(device=dev)
    g.manual_seed(SEED)
    xa = torch.randn((rows, H), generator=g, device=dev).to(torch.bfloat16)
    a_codes, a_scales = ops.mx_quant(xa, "E4M3", "rne")
    del xa
    w1, w1s = quant_weights(E, N, H, 0.02, SEED + 1)
    act_codes = torch.empty((rows, N // 2), dtype=torch.uint8, device=dev)
    act_scales = torch.empty((rows, ops.scale_cols(N // 2)), dtype=torch.uint8, device=dev)
    gws = ops.gmm_workspace(E, dev)

    def step():
        ops.mx_gmm_swiglu_quant(a_codes, a_scales, w1, w1s, counts, H, workspace=gws, outs=(act_codes, act_scales))

    def time_headline():
        """One timed region, measured twice: host clock bracketed by synchronize (-> value) and HIP events recorded
        on the launch stream around the same K launches (-> roofline.achieved)."""
        for _ in range(WARM):
            step()
        torch.cuda.synchronize()
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(K_STEPS):
            step()
        ev1.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / K_STEPS, ev0.elapsed_time(ev1) * 1e-3 / K_STEPS

    flop = 2.0 * rows * H * N

    # ------------------------------------------------------------------ in-run correctness check ----
    # Before anything is timed: the benchmarked instantiation (no bf16 output) must give the same codes and scales as
    # the one that also writes the bf16 SwiGLU values, on every row; those must be what the stand-alone quantizer
    # makes of that bf16 output; and on sampled rows of the largest expert the bf16 values must agree with the CPU
    # oracle's golden chain (rtol 2e-2) and the codes with the oracle quantizer, bit for bit.
    step()
    chk_codes, chk_scales, chk_act = ops.mx_gmm_swiglu_quant(a_codes, a_scales, w1, w1s, counts, H, want_bf16=True)
    if not (torch.equal(chk_codes, act_codes) and torch.equal(chk_scales, act_scales)):
        log("bench.py: the benchmarked kernel disagrees with its bf16-output variant")
        return 4
    hq, hs = ops.mx_quant(chk_act, "E4M3", "rne")
    if not (torch.equal(hq, act_codes) and torch.equal(hs, act_scales)):
        log("bench.py: requantised codes are not what the quantizer makes of the kernel's bf16 output")
        return 4
    if not args.no_cpu:
        from oracle import mx_oracle as O
        e_big = int(np.argmax(counts_h))
        off_h = np.concatenate([[0], np.cumsum(counts_h)])
        pick = off_h[e_big] + np.array([0, 1, counts_h[e_big] // 2, counts_h[e_big] - 1])
        pk = torch.from_numpy(pick).to(dev)
        _, act_g, _, _ = O.gmm1_swiglu_quant(a_codes[pk].cpu().numpy(), a_scales[pk].cpu().numpy(), w1[e_big:e_big + 1].cpu().numpy(),
                                             w1s[e_big:e_big + 1].cpu().numpy(), [len(pick)])
        got_act = chk_act[pk].view(torch.int16).cpu().numpy().view(np.uint16)
        gold_act = O.bf16_bits_to_f32(act_g)
        err = np.abs(O.bf16_bits_to_f32(got_act) - gold_act)
        oq, osc = O.mx_quant_bf16(got_act, "E4M3", "rne")
        if (err > 1e-3 + 2e-2 * np.abs(gold_act)).any() or not np.array_equal(oq, act_codes[pk].cpu().numpy()) \
                or not np.array_equal(osc, act_scales[pk].cpu().numpy()):
            log(f"bench.py: sampled rows disagree with the CPU oracle (max abs err {err.max():.4g})")
            return 4
        log(f"[check] codes/scales identical across instantiations and to the quantizer on all {rows} rows; "
            f"4 sampled rows vs CPU oracle: max abs err {err.max():.3g}")
    del chk_codes, chk_scales, chk_act, hq, hs

    # ------------------------------------------------------------------ extras -----------------
    extra = {}
    want = set(x for x in args.only.split(",") if x) or {"quant", "gemm", "ffn", "fp4", "int8", "routing", "idle"}
    if args.no_extras:
        want = set()

    if "copycal" in want:
        # plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run
        nbytes = 1 << 30
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        tcopy = hip_time(lambda: dst.copy_(src), steps=5, warm=1)
        extra["copycal"] = {"bytes_read": nbytes, "bytes_written": nbytes, "avg_launch_us": tcopy * 1e6,
                            "GBs": 2 * nbytes / tcopy / 1e9}
        log(f"[copy calibration] 1 GiB -> 1 GiB in {tcopy*1e6:.1f} us = {2*nbytes/tcopy/1e9:.0f} GB/s")
        # what the memory system gives a write-only and a read-only stream of the same size (torch's fill and
        # reduction kernels): the practical ceilings next to which the write-heavy scatter and the read-heavy
        # combine are to be read
        tfill = hip_time(lambda: dst.zero_(), steps=5, warm=1)
        src32 = src.view(torch.int32)
        tread = hip_time(lambda: torch.max(src32), steps=5, warm=1)
        extra["copycal"].update({"write_only_GBs": nbytes / tfill / 1e9, "read_only_GBs": nbytes / tread / 1e9})
        log(f"[ceilings] write-only {nbytes/tfill/1e9:.0f} GB/s, read-only {nbytes/tread/1e9:.0f} GB/s")
        del src, dst, src32

    if "quant" in want:
        M1, K1 = 4096, 7168
        x1 = torch.from_numpy(W.activations_with_outliers(M1, K1, SEED).view(np.int16)).to(dev)
        q1 = torch.empty((M1, K1), dtype=torch.uint8, device=dev)
        s1 = torch.empty((M1, K1 // 32), dtype=torch.uint8, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        tq = hip_time(lambda: lib.cmx_mx_quant(x1.data_ptr(), K1, q1.data_ptr(), K1, s1.data_ptr(), K1 // 32, M1, K1, 0, 0, st),
                      steps=max(K_STEPS, 50))
        bytes_q = M1 * K1 * 2 + M1 * K1 + M1 * K1 // 32
        extra["mx_quant_cfg1"] = {"kernel": "mx_quant_rne8_kernel<E4M3>", "bound": "hbm", "achieved": bytes_q / tq / 1e9,
                                  "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_q / tq / 1e9 / HBM_PEAK_GBS,
                                  "bytes_per_launch": bytes_q, "avg_launch_us": tq * 1e6, "traffic": None}
        log(f"[mx_quant cfg1] {tq*1e6:.1f} us -> {bytes_q/tq/1e9:.0f} GB/s")
        del x1, q1, s1

    if "gemm" in want:
        M2, N2, K2 = 8192, 4096, 7168
        g.manual_seed(SEED + 2)
        a2, a2s = ops.mx_quant(torch.randn((M2, K2), generator=g, device=dev).to(torch.bfloat16))
        b2, b2s = ops.mx_quant(torch.randn((N2, K2), generator=g, device=dev).to(torch.bfloat16))
        tg = hip_time(lambda: ops.mx_gemm(a2, a2s, b2, b2s, K2))
        fl2 = 2.0 * M2 * N2 * K2
        extra["mx_gemm_cfg2"] = {"kernel": "mx_gemm_pipe_kernel<E4M3, store epilogue, 256x256 tile, 2x2 wavefronts> (dense)", "bound": "mfma",
                                 "achieved": fl2 / tg / 1e12, "peak": MXFP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                                 "frac": fl2 / tg / 1e12 / MXFP8_PEAK_TFLOPS, "avg_launch_us": tg * 1e6}
        log(f"[mx_gemm cfg2] {tg*1e6:.1f} us -> {fl2/tg/1e12:.0f} TFLOP/s")
        # the same B stored [K, N] with scales [K/64, N, 2]: the layout pass alone (one read + one write of B)
        bt = b2.t().contiguous()
        bts = b2s.reshape(N2, K2 // 64, 2).permute(1, 0, 2).contiguous()
        bk = torch.empty((N2, K2), dtype=torch.uint8, device=dev)
        bks = torch.empty((N2, K2 // 32), dtype=torch.uint8, device=dev)
        st2 = torch.cuda.current_stream().cuda_stream
        tl = hip_time(lambda: lib.cmx_mx_to_k_major(bt.data_ptr(), N2, bts.data_ptr(), bk.data_ptr(), K2, bks.data_ptr(), K2 // 32,
                                                    K2, N2, 1, st2))
        bytes_l = 2 * (N2 * K2 + N2 * K2 // 32)
        # a 30 MB operand is gone in a dozen microseconds: a plain device copy of the same bytes is the yardstick there;
        # the sixteen experts of config 3's W1 (485 MB) show the rate of the kernel itself
        flat = torch.empty(bytes_l // 2, dtype=torch.uint8, device=dev)
        flat2 = torch.empty_like(flat)
        tcp = hip_time(lambda: flat2.copy_(flat))
        wt = torch.empty((E, H, N), dtype=torch.uint8, device=dev)
        wts = torch.empty((E, H // 64, N, 2), dtype=torch.uint8, device=dev)
        wk = torch.empty((E, N, H), dtype=torch.uint8, device=dev)
        wks = torch.empty((E, N, H // 32), dtype=torch.uint8, device=dev)
        tlw = hip_time(lambda: lib.cmx_mx_to_k_major(wt.data_ptr(), N, wts.data_ptr(), wk.data_ptr(), H, wks.data_ptr(), H // 32,
                                                     H, N, E, st2), steps=max(5, K_STEPS // 2))
        bytes_w = 2 * E * (N * H + N * H // 32)
        extra["mx_to_k_major_cfg2_B"] = {"kernel": "mx_to_k_major16_kernel", "bound": "hbm", "achieved": bytes_l / tl / 1e9,
                                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_l / tl / 1e9 / HBM_PEAK_GBS,
                                         "bytes_per_launch": bytes_l, "avg_launch_us": tl * 1e6,
                                         "device_copy_of_the_same_bytes_us": tcp * 1e6}
        extra["mx_to_k_major_cfg3_W1"] = {"kernel": "mx_to_k_major16_kernel", "bound": "hbm", "achieved": bytes_w / tlw / 1e9,
                                          "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bytes_w / tlw / 1e9 / HBM_PEAK_GBS,
                                          "bytes_per_launch": bytes_w, "avg_launch_us": tlw * 1e6}
        log(f"[mx_to_k_major cfg2 B] {tl*1e6:.1f} us -> {bytes_l/tl/1e9:.0f} GB/s (copy of the same bytes {tcp*1e6:.1f} us); "
            f"cfg3 W1 {tlw*1e6:.1f} us -> {bytes_w/tlw/1e9:.0f} GB/s")
        del bk, bks, flat, flat2, wt, wts, wk, wks
        del a2, a2s, b2, b2s, bt, bts

    if "int8" in want:
        # the reference operator's own arithmetic (INT8 W8A8, per-channel and per-token scales) at config 3's shape
        g.manual_seed(SEED + 8)
        a8 = torch.randint(-127, 128, (rows, H), dtype=torch.int8, device=dev, generator=g)
        ts8 = torch.rand((rows,), device=dev, generator=g) * 1e-2 + 1e-3
        w8 = torch.randint(-127, 128, (E, N, H), dtype=torch.int8, device=dev, generator=g)      # [E, N, K]: K-contiguous
        ch8 = torch.rand((E * N,), device=dev, generator=g) * 1e-4
        o8 = torch.empty((rows, N // 2), dtype=torch.float32, device=dev)
        t8 = hip_time(lambda: ops.int8_gmm_dequant_swiglu(a8, ts8, w8, ch8, counts, N, H, 1, "fp32", c=o8))
        extra["int8_gmm_dequant_swiglu_cfg3_shape"] = {
            "kernel": "mx_gemm_dl_kernel<INT8, dequant+swiglu epilogue, 256x256 tile, 8 wavefronts> (grouped)", "bound": "mfma",
            "achieved": flop / t8 / 1e12, "peak": INT8_PEAK_TOPS, "unit": "TOP/s", "frac": flop / t8 / 1e12 / INT8_PEAK_TOPS,
            "avg_launch_us": t8 * 1e6}
        log(f"[int8 gmm+dequant+swiglu, cfg3 shape] {t8*1e6:.1f} us -> {flop/t8/1e12:.0f} TOP/s")
        w8t = w8.transpose(1, 2).contiguous()                                                   # [E, K, N] as the reference stores it
        t8b = hip_time(lambda: ops.int8_gmm_dequant_swiglu(a8, ts8, w8t, ch8, counts, N, H, 0, "fp32", c=o8), steps=max(5, K_STEPS // 4))
        extra["int8_gmm_dequant_swiglu_cfg3_shape"]["avg_launch_us_k_slow_weights"] = t8b * 1e6
        log(f"[int8, weights stored [E,K,N] and rewritten per call] {t8b*1e6:.1f} us")
        del a8, ts8, w8, w8t, ch8, o8

    if "fp4" in want:
        E5, T5, K5, N5 = 32, 8192, 7168, 4096
        idx5 = W.zipf_routing(T5, E5, 8, SEED + 5)
        c5h = np.bincount(idx5.reshape(-1), minlength=E5).astype(np.int32)
        rows5 = int(c5h.sum())
        c5 = torch.from_numpy(c5h).to(dev)
        g.manual_seed(SEED + 5)
        a5, a5s = ops.mx_quant((torch.rand((rows5, K5), generator=g, device=dev) * 4 - 2).to(torch.bfloat16), "E2M1", "lut")
        w5 = torch.empty((E5, N5, K5 // 2), dtype=torch.uint8, device=dev)
        w5s = torch.empty((E5, N5, K5 // 32), dtype=torch.uint8, device=dev)
        for i in range(E5):
            q, s = ops.mx_quant((torch.rand((N5, K5), generator=g, device=dev) * 4 - 2).to(torch.bfloat16), "E2M1", "lut")
            w5[i], w5s[i] = q, s
        c_out = torch.empty((rows5, N5), dtype=torch.bfloat16, device=dev)
        ws5 = ops.gmm_workspace(E5, dev)
        t5 = hip_time(lambda: ops.mx_gmm(a5, a5s, w5, w5s, c5, K5, "E2M1", "bf16", c=c_out, workspace=ws5))
        fl5 = 2.0 * rows5 * K5 * N5
        extra["mxfp4_gmm_cfg5"] = {"kernel": "mx_gemm_pipe_fp4_kernel<bf16 store epilogue, 2x2 wavefronts, persistent> (grouped, 256x256 tile)", "bound": "mfma",
                                   "achieved": fl5 / t5 / 1e12, "peak": MXFP4_PEAK_TFLOPS, "unit": "TFLOP/s",
                                   "frac": fl5 / t5 / 1e12 / MXFP4_PEAK_TFLOPS, "avg_launch_us": t5 * 1e6}
        log(f"[mxfp4 gmm cfg5] {t5*1e6:.1f} us -> {fl5/t5/1e12:.0f} TFLOP/s")
        del a5, a5s, w5, w5s, c_out

    if "ffn" in want or "routing" in want:
        T4, E4, K4, N4, TOP4 = 8192, 256, 7168, 4096, 8
        idx4, p4 = W.softmax_topk_routing(T4, E4, TOP4, SEED + 4)
        idx4_d, p4_d = torch.from_numpy(idx4).to(dev), torch.from_numpy(p4).to(dev)
        g.manual_seed(SEED + 4)
        x4 = torch.randn((T4, K4), generator=g, device=dev).to(torch.bfloat16)
        rows4 = T4 * TOP4
        if "routing" in want:
            s2s, inv, cnt4 = ops.moe_init_routing(idx4_d, E4)
            ts = hip_time(lambda: ops.moe_init_routing(idx4_d, E4))
            qa = torch.empty((rows4, K4), dtype=torch.uint8, device=dev)
            # scale rows at the pitch the FFN chain uses (whole 128-byte lines: 256 bytes for K/32 = 224 scale bytes)
            sp4 = ops.ffn_workspace_layout(T4, K4, N4, E4, TOP4)["a_scales_pitch"]
            qs = torch.empty((rows4, sp4), dtype=torch.uint8, device=dev)
            st = torch.cuda.current_stream().cuda_stream
            tqs = hip_time(lambda: lib.cmx_quant_scatter(x4.data_ptr(), K4, inv.data_ptr(), qa.data_ptr(), K4, qs.data_ptr(),
                                                         sp4, T4, K4, TOP4, st))
            b_qs = T4 * K4 * 2 + rows4 * (K4 + K4 // 32)
            y4 = torch.randn((rows4, K4), generator=g, device=dev).to(torch.bfloat16)
            tc4 = hip_time(lambda: ops.moe_token_unpermute(y4, inv, p4_d))
            b_c = rows4 * K4 * 2 + T4 * K4 * 2

            def spaced(fn, reps=8):
                """Average duration (s) of single launches of fn() that each follow a launch of the headline matmul
                instead of a copy of themselves (HIP events around every launch)."""
                tot = 0.0
                for r in range(reps + 2):
                    step()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    fn()
                    e1.record()
                    torch.cuda.synchronize()
                    if r >= 2:
                        tot += e0.elapsed_time(e1) * 1e-3 / reps
                return tot

            # back to back, a kernel that writes 486 MB competes with the write-back of its predecessor's lines (the
            # memory-side cache still holds them); inside the FFN chain it follows a matmul that leaves HBM bandwidth
            # free.  "frac" is the sustained back-to-back rate, "frac_after_matmul" the rate of a launch placed as in
            # the chain.
            tqs_sp = spaced(lambda: lib.cmx_quant_scatter(x4.data_ptr(), K4, inv.data_ptr(), qa.data_ptr(), K4, qs.data_ptr(),
                                                          sp4, T4, K4, TOP4, st))
            tc4_sp = spaced(lambda: ops.moe_token_unpermute(y4, inv, p4_d))
            extra["routing_cfg4"] = {
                "expert_sort_us": ts * 1e6,
                "quant_scatter": {"bound": "hbm", "achieved": b_qs / tqs / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": b_qs / tqs / 1e9 / HBM_PEAK_GBS, "avg_launch_us": tqs * 1e6,
                                  "after_matmul_us": tqs_sp * 1e6, "frac_after_matmul": b_qs / tqs_sp / 1e9 / HBM_PEAK_GBS},
                "unpermute_combine": {"bound": "hbm", "achieved": b_c / tc4 / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                      "frac": b_c / tc4 / 1e9 / HBM_PEAK_GBS, "avg_launch_us": tc4 * 1e6,
                                      "after_matmul_us": tc4_sp * 1e6, "frac_after_matmul": b_c / tc4_sp / 1e9 / HBM_PEAK_GBS}}
            log(f"[routing cfg4] sort {ts*1e6:.1f} us, quant_scatter {b_qs/tqs/1e9:.0f} GB/s, combine {b_c/tc4/1e9:.0f} GB/s")
            del qa, qs, y4
        if "ffn" in want:
            w14, w14s = quant_weights(E4, N4, K4, 0.02, SEED + 6)
            w24, w24s = quant_weights(E4, K4, N4 // 2, 0.02, SEED + 7)
            wsp = torch.empty(ops.ffn_workspace_bytes(T4, K4, N4, E4, TOP4), dtype=torch.uint8, device=dev)
            out4 = torch.empty((T4, K4), dtype=torch.bfloat16, device=dev)
            tf = hip_time(lambda: ops.dispatch_ffn_combine(x4, idx4_d, p4_d, w14, w14s, w24, w24s, workspace=wsp, out=out4),
                          steps=max(5, K_STEPS // 2), warm=2)
            fl4 = 2.0 * rows4 * K4 * (N4 + N4 // 2)
            by4 = float(w14.numel() + w14s.numel() + w24.numel() + w24s.numel()) + T4 * K4 * 2 \
                + 2 * rows4 * (K4 + K4 // 32) + 2 * rows4 * (N4 // 2 + N4 // 64) + 2 * rows4 * K4 * 2 + T4 * K4 * 2
            # the same chain stage by stage (the C entry points the FFN calls, in its order, on its kind of buffers),
            # HIP events between the stages: what each kernel takes inside the chain, where it follows other work
            # instead of a copy of itself
            lay4 = ops.ffn_workspace_layout(T4, K4, N4, E4, TOP4)
            sp = lay4["a_scales_pitch"]
            ac = torch.empty((rows4, K4), dtype=torch.uint8, device=dev)
            asc = torch.empty((rows4, sp), dtype=torch.uint8, device=dev)
            hc = torch.empty((rows4, N4 // 2), dtype=torch.uint8, device=dev)
            hs = torch.empty((rows4, ops.scale_cols(N4 // 2)), dtype=torch.uint8, device=dev)
            yy = torch.empty((rows4, K4), dtype=torch.bfloat16, device=dev)
            gw1, gw2 = ops.gmm_workspace(E4, dev), ops.gmm_workspace(E4, dev)
            st4 = torch.cuda.current_stream().cuda_stream
            names = ["expert_sort", "quant_scatter", "gmm1_swiglu_requant", "gmm2", "unpermute_combine"]
            acc_ms = [0.0] * 5
            reps = max(3, K_STEPS // 4)
            for rep in range(reps + 2):
                evs = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
                evs[0].record()
                s2s4, inv4, cnt4b = ops.moe_init_routing(idx4_d, E4)
                evs[1].record()
                lib.cmx_quant_scatter(x4.data_ptr(), K4, inv4.data_ptr(), ac.data_ptr(), K4, asc.data_ptr(), sp, T4, K4, TOP4, st4)
                evs[2].record()
                ops.mx_gmm_swiglu_quant(ac, asc, w14, w14s, cnt4b, K4, workspace=gw1, outs=(hc, hs))
                evs[3].record()
                ops.mx_gmm(hc, hs, w24, w24s, cnt4b, N4 // 2, "E4M3", "bf16", c=yy, workspace=gw2)
                evs[4].record()
                ops.moe_token_unpermute(yy, inv4, p4_d)
                evs[5].record()
                torch.cuda.synchronize()
                if rep >= 2:
                    for i in range(5):
                        acc_ms[i] += evs[i].elapsed_time(evs[i + 1]) / reps
            b_qs4 = T4 * K4 * 2 + rows4 * (K4 + K4 // 32)
            b_c4 = rows4 * K4 * 2 + T4 * K4 * 2
            stages = {n: {"us": acc_ms[i] * 1e3} for i, n in enumerate(names)}
            stages["quant_scatter"].update({"hbm_frac": b_qs4 / (acc_ms[1] * 1e-3) / 1e9 / HBM_PEAK_GBS})
            stages["unpermute_combine"].update({"hbm_frac": b_c4 / (acc_ms[4] * 1e-3) / 1e9 / HBM_PEAK_GBS})
            log("[moe ffn cfg4 stages] " + ", ".join(f"{n} {v['us']:.0f} us" for n, v in stages.items()))
            # the same chain on weights pre-tiled once at load time (cmx_mx_pretile_weights): both matmuls then run the
            # weights-to-registers kernel
            t0 = time.perf_counter()
            w14t, w24t = ops.pretile_weights(w14, True), ops.pretile_weights(w24, False)
            torch.cuda.synchronize()
            t_tile = time.perf_counter() - t0
            tft = hip_time(lambda: ops.dispatch_ffn_combine(x4, idx4_d, p4_d, w14t, w14s, w24t, w24s, workspace=wsp, out=out4),
                           steps=max(5, K_STEPS // 2), warm=2)
            tg1 = hip_time(lambda: ops.mx_gmm_swiglu_quant(ac, asc, w14t, w14s, cnt4b, K4, workspace=gw1, outs=(hc, hs)), steps=5, warm=2)
            tg2 = hip_time(lambda: ops.mx_gmm(hc, hs, w24t, w24s, cnt4b, N4 // 2, "E4M3", "bf16", c=yy, workspace=gw2), steps=5, warm=2)
            rate = lambda t: {"ms": t * 1e3, "tflops": fl4 / t / 1e12, "mfma_frac": fl4 / t / 1e12 / MXFP8_PEAK_TFLOPS,
                              "hbm_GBs": by4 / t / 1e9, "hbm_frac": by4 / t / 1e9 / HBM_PEAK_GBS, "tokens_per_s": T4 / t}
            log(f"[moe ffn cfg4, pre-tiled weights] {tft*1e3:.3f} ms (gmm1 {tg1*1e6:.0f} us, gmm2 {tg2*1e6:.0f} us back to back; tiling pass once {t_tile*1e3:.1f} ms)")
            del ac, asc, hc, hs, yy, w14t, w24t
            # "ms": the chain as the operator layer runs it (its weights are tiled where it loads them); the reference's
            # own entry point on row-major weights, with its stages, under "row_major_weights"
            extra["moe_ffn_cfg4"] = {**rate(tft),
                                     "weights": "pre-tiled once at load time (cmx_mx_pretile_weights), as the host operator Ascend950DispatchFFNCombine keeps them",
                                     "entry": "cmx_dispatch_ffn_combine_pretiled", "gmm1_swiglu_requant_us": tg1 * 1e6, "gmm2_us": tg2 * 1e6,
                                     "pretile_pass_ms_once": t_tile * 1e3, "algorithmic_GB": by4 / 1e9,
                                     "row_major_weights": {**rate(tf), "entry": "catccos_ascend950_dispatch_ffn_combine", "stages_in_chain": stages}}
            log(f"[moe ffn cfg4, row-major weights] {tf*1e3:.3f} ms -> {fl4/tf/1e12:.0f} TFLOP/s, {by4/tf/1e9:.0f} GB/s algorithmic")

    # ------------------------------------------------------------------ headline timing ---------
    # The extras above ran first, so this is a GPU that has been busy, as it is in a training or serving job.  (After
    # an idle period the first ~25 launches of an MFMA-bound kernel run up to 30 % slower while the power management
    # settles: extra.after_idle records that case.)
    wall, kern = time_headline()
    value = flop / wall / 1e12
    log(f"[gmm1+swiglu+requant cfg3] wall {wall*1e6:.1f} us/step, events {kern*1e6:.1f} us -> {flop/kern/1e12:.0f} TFLOP/s")
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic_config3.json")
    if os.path.exists(tpath):
        # HBM-side bytes per launch from the rocprofv3 --pmc runs summarised next to that file (FETCH_SIZE and
        # WRITE_SIZE scaled by what the same counters read for a 1 GiB copy); profiled, not measured in this run
        with open(tpath) as f:
            traffic = json.load(f).get("traffic_bytes_per_launch")
    roofline = {"kernel": "mx_gemm_pipe_kernel<E4M3, swiglu+requant epilogue, 256x256 tile, 2x2 wavefronts, persistent> (grouped, config 3; one launch also runs the 1-workgroup gmm_prepare_kernel)", "bound": "mfma",
                "achieved": flop / kern / 1e12, "peak": MXFP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": flop / kern / 1e12 / MXFP8_PEAK_TFLOPS, "traffic": traffic,
                "flop_per_launch": flop, "avg_launch_us": kern * 1e6}
    value_after_idle = None
    if "idle" in want:
        time.sleep(3.0)
        w_idle, k_idle = time_headline()
        value_after_idle = flop / w_idle / 1e12
        extra["after_idle"] = {"idle_s": 3.0, "warmup": WARM, "steps": K_STEPS, "avg_launch_us": k_idle * 1e6,
                               "note": "the same timed region started 3 s after the GPU went idle"}
        log(f"[after 3 s idle] events {k_idle*1e6:.1f} us")

    # ------------------------------------------------------------------ CPU baseline -----------
    cpu = None
    if not args.no_cpu:
        from oracle import mx_oracle as O
        sample_groups = [int(i) for i in np.argsort(-counts_h)[:8]]     # the 8 largest experts, up to 2048 rows each
        cap = 2048
        off = np.concatenate([[0], np.cumsum(counts_h)])
        a_h, as_h = [], []
        cnt = []
        for gi in sample_groups:
            r = min(cap, int(counts_h[gi]))
            a_h.append(a_codes[off[gi]:off[gi] + r].cpu().numpy())
            as_h.append(a_scales[off[gi]:off[gi] + r].cpu().numpy())
            cnt.append(r)
        a_h, as_h = np.concatenate(a_h), np.concatenate(as_h)
        w_h = w1[sample_groups].cpu().numpy()
        ws_h = w1s[sample_groups].cpu().numpy()
        O.gmm1_swiglu_quant(a_h[:64], as_h[:64], w_h[:2], ws_h[:2], [32, 32])        # warm-up
        reps = []
        for _ in range(3):
            t0 = time.perf_counter()
            O.gmm1_swiglu_quant(a_h, as_h, w_h, ws_h, cnt)
            reps.append(time.perf_counter() - t0)
        tc = float(np.median(reps))
        cflop = 2.0 * sum(cnt) * H * N
        cores = len(os.sched_getaffinity(0))
        omp = os.environ.get("OMP_NUM_THREADS")
        if omp and omp.isdigit():
            cores = min(cores, int(omp))
        cpu = {"value": cflop / tc / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
               "sample": f"numpy oracle gmm1_swiglu_quant on {len(cnt)} experts x {cnt} rows (K={H}, N={N}), "
                         f"median of 3 = {tc:.2f} s; includes dequantising operands to fp32"}
        log(f"[cpu baseline] {cpu['value']*1e3:.1f} GFLOP/s on {cores} threads ({tc:.2f} s)")
        del a_h, as_h, w_h, ws_h

    line = {
        "metric": "MXFP8 GMM TFLOP/s (% MFMA peak); MX-quant GB/s (% HBM peak), 1 GPU",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": K_STEPS, "warmup": WARM,
        "ms_per_step": wall * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp8 (E4M3 elements, E8M0 block-32 scales), fp32 accumulate", "data": "synthetic",
        "config": {"workload": "config 3: MoE grouped matmul + dequant + SwiGLU + MX requant, E=16, 4096 tokens x top-8 "
                               "Zipf(1.1) routed (2 empty experts), H=7168, W [16,4096,7168] MXFP8",
                   "rows": rows, "K": H, "N": N, "experts": E, "seed": SEED,
                   "group_sizes": counts_h.tolist()},
        "mfma_peak_frac": value / MXFP8_PEAK_TFLOPS,
        # the same timed region started 3 s after the GPU went idle (no extras in front of it): the figure that is
        # comparable with runs that time the headline first, on a chip whose clock has not settled
        "value_after_idle": value_after_idle,
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
