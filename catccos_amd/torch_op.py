"""`torch.ops.catccos.*` on PyTorch-ROCm, one GPU.

Mirrors the op surface of the reference's torch binding
(examples/torch_binding/src/torch_bindings.cpp:109-151 init, :213-325 ascend950_dispatch_ffn_combine,
:328-365 finalize, schemas :369-387): same op names, argument order, dtypes, shape rules and error
messages where they make sense without NPUs and shmem.  Importing this module registers the ops;
the compute is the C-ABI entry point `catccos_ascend950_dispatch_ffn_combine`, nothing else.

    import catccos_amd.torch_op
    torch.ops.catccos.init(0, 1, 1 << 30, "tcp://127.0.0.1:1")
    y = torch.ops.catccos.ascend950_dispatch_ffn_combine(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale)
    torch.ops.catccos.finalize()

Tensor contract: x bf16 [M, K]; expert_idx int32 / gate_weight fp32 [M, TopK]; w1 float8_e4m3fn [E, N, K],
w1_scale float8_e8m0fnu [E, N, K/32]; w2 float8_e4m3fn [E, K, N/2], w2_scale float8_e8m0fnu [E, K, N/64];
result bf16 [M, K].  The workspace is allocated on first use and kept until finalize(), as the reference
keeps `state.workspace`.

Two ops beyond the reference's surface serve the pre-tiled weight layout of this library (K % 512 == 0, N % 1024 == 0):

    w1_tiled, w2_tiled = torch.ops.catccos.ascend950_pretile_ffn_weights(w1, w2)        # once, when the weights are loaded
    y = torch.ops.catccos.ascend950_dispatch_ffn_combine_pretiled(x, expert_idx, gate_weight, w1_tiled, w1_scale,
                                                                  w2_tiled, w2_scale)   # same bits as the op above

w1_tiled / w2_tiled are flat uint8 tensors (cmx_mx_pretile_weights); the shapes come from the scale tensors.
"""
from __future__ import annotations

import torch

from . import _lib

_state = {"initialized": False, "rank_id": -1, "rank_size": 0, "device": None, "workspace": None}

_lib_def = torch.library.Library("catccos", "DEF")
_lib_def.define("init(int rank_id, int rank_size, int local_mem_size, str ip_port) -> int")
_lib_def.define("ascend950_dispatch_ffn_combine(Tensor x, Tensor expert_idx, Tensor gate_weight, "
                "Tensor w1, Tensor w1_scale, Tensor w2, Tensor w2_scale) -> Tensor")
_lib_def.define("finalize() -> int")
_lib_def.define("ascend950_pretile_ffn_weights(Tensor w1, Tensor w2) -> Tensor[]")
_lib_def.define("ascend950_dispatch_ffn_combine_pretiled(Tensor x, Tensor expert_idx, Tensor gate_weight, "
                "Tensor w1_tiled, Tensor w1_scale, Tensor w2_tiled, Tensor w2_scale) -> Tensor")


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _init(rank_id: int, rank_size: int, local_mem_size: int, ip_port: str) -> int:
    if _state["initialized"]:
        _check(rank_id == _state["rank_id"] and rank_size == _state["rank_size"],
               "CatCCOS is already initialized with a different rank configuration")
        return 0
    _check(rank_id >= 0, f"invalid rank_id: {rank_id}")
    _check(rank_size > 0, f"invalid rank_size: {rank_size}")
    _check(rank_id < rank_size and rank_size <= 2 ** 31 - 1, "invalid rank configuration")
    _check(local_mem_size > 0, f"invalid local_mem_size: {local_mem_size}")
    _check(len(ip_port) > 0, "ip_port is empty")
    _check(rank_size == 1, "this build runs one rank per process without collectives: rank_size must be 1")
    _check(torch.cuda.is_available(), "no GPU visible")
    _lib.load()                                   # fails loudly when the HIP library is missing
    _state.update(initialized=True, rank_id=rank_id, rank_size=rank_size,
                  device=torch.device("cuda", torch.cuda.current_device()), workspace=None)
    return 0


def _finalize() -> int:
    if not _state["initialized"]:
        return 0
    torch.cuda.synchronize(_state["device"])
    _state.update(initialized=False, rank_id=-1, rank_size=0, device=None, workspace=None)
    return 0


def _pretile(w1, w2):
    _check(_state["initialized"], "call torch.ops.catccos.init(...) first")
    _check(w1.dim() == 3 and w2.dim() == 3 and w1.dtype == torch.float8_e4m3fn and w2.dtype == torch.float8_e4m3fn,
           "w1 and w2 must be 3D float8_e4m3fn tensors")
    _check(w1.is_cuda and w2.device == w1.device and w1.is_contiguous() and w2.is_contiguous(), "w1 and w2 must be contiguous GPU tensors")
    e, n, k = w1.shape
    _check(tuple(w2.shape) == (e, k, n // 2), "invalid w2 shape")
    _check(k % 512 == 0 and n % 1024 == 0, "pre-tiled weights need K divisible by 512 and N by 1024")
    lib = _lib.load()
    stream = torch.cuda.current_stream(w1.device).cuda_stream
    outs = []
    for w, rows, cols, pair in ((w1, n, k, 1), (w2, k, n // 2, 0)):
        t = torch.empty(lib.cmx_mx_pretiled_weight_bytes(e, rows, cols, pair), dtype=torch.uint8, device=w.device)
        _lib.check(lib.cmx_mx_pretile_weights(w.data_ptr(), t.data_ptr(), e, rows, cols, pair, stream))
        for u in (w, t):
            u.record_stream(torch.cuda.current_stream(w.device))
        outs.append(t)
    return outs


def _ffn(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale):
    return _ffn_any(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale, False)


def _ffn_pretiled(x, expert_idx, gate_weight, w1_tiled, w1_scale, w2_tiled, w2_scale):
    return _ffn_any(x, expert_idx, gate_weight, w1_tiled, w1_scale, w2_tiled, w2_scale, True)


def _ffn_any(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale, tiled):
    _check(_state["initialized"], "call torch.ops.catccos.init(...) first")
    _check(x.device == _state["device"], "CatCCOS must run on its initialized device")
    wt, wd = (torch.uint8, 1) if tiled else (torch.float8_e4m3fn, 3)
    inputs = ((x, "x", torch.bfloat16, 2), (expert_idx, "expert_idx", torch.int32, 2), (gate_weight, "gate_weight", torch.float32, 2),
              (w1, "w1", wt, wd), (w1_scale, "w1_scale", torch.float8_e8m0fnu, 3),
              (w2, "w2", wt, wd), (w2_scale, "w2_scale", torch.float8_e8m0fnu, 3))
    for t, name, dtype, dims in inputs:
        _check(t.device == x.device, f"{name} must be on the same device as x")
        _check(t.dtype == dtype, f"{name} must have dtype {dtype}")
        _check(t.dim() == dims, f"{name} must be {dims}D")
        _check(t.is_contiguous(), f"{name} must have contiguous strides")
    m, k = x.shape
    n = w1_scale.shape[1]
    top_k, local_experts, rank_size = expert_idx.shape[1], w1_scale.shape[0], _state["rank_size"]
    _check(m > 0 and k > 0 and n > 0, "M, K and N must be positive")
    _check(k <= 0xFFFFFFFF and n <= 0xFFFFFFFF, "K or N exceeds the uint32 kernel limit")
    _check(k % 256 == 0 and n % 512 == 0, "K must be divisible by 256 and N by 512")
    _check(0 < local_experts <= (2 ** 31 - 1) // rank_size, "total expert count exceeds the int32 kernel limit")
    _check(0 < top_k <= local_experts * rank_size, "invalid TopK")
    _check(top_k <= 64, "TopK exceeds the weighted combine's limit of 64")
    _check(m <= (2 ** 31 - 1) // rank_size // top_k, "routed row count exceeds the int32 kernel limit")
    k2, scale_k, scale_k2 = n // 2, k // 32, n // 64
    _check(expert_idx.shape[0] == m and gate_weight.shape == expert_idx.shape, "expected [M, TopK] routing")
    lib = _lib.load()
    if tiled:
        _check(k % 512 == 0 and n % 1024 == 0, "pre-tiled weights need K divisible by 512 and N by 1024")
        _check(w1.numel() == lib.cmx_mx_pretiled_weight_bytes(local_experts, n, k, 1), "w1_tiled has the wrong size for w1_scale's shape")
        _check(w2.numel() == lib.cmx_mx_pretiled_weight_bytes(local_experts, k, k2, 0), "w2_tiled has the wrong size for w2_scale's shape")
    else:
        _check(tuple(w1.shape) == (local_experts, n, k), "w1 must have shape [local_experts, N, K]")
        _check(tuple(w2.shape) == (local_experts, k, k2), "invalid w2 shape")
    _check(tuple(w1_scale.shape) == (local_experts, n, scale_k), "invalid w1_scale shape")
    _check(tuple(w2_scale.shape) == (local_experts, k, scale_k2), "invalid w2_scale shape")

    need = lib.catccos_ascend950_dispatch_ffn_combine_workspace_bytes(m, k, n, local_experts, top_k, rank_size)
    ws = _state["workspace"]
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        _state["workspace"] = ws
    out = torch.empty((m, k), dtype=torch.bfloat16, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    ptr = lambda t: t.data_ptr()
    if tiled:
        _lib.check(lib.cmx_dispatch_ffn_combine_pretiled(
            stream, ptr(x), ptr(expert_idx), ptr(gate_weight), ptr(w1), ptr(w1_scale), ptr(w2), ptr(w2_scale), ptr(out),
            ptr(ws), m, k, n, local_experts, top_k))
    else:
        _lib.check(lib.catccos_ascend950_dispatch_ffn_combine(
            0, stream, 0, ptr(x), ptr(expert_idx), ptr(gate_weight), ptr(w1), ptr(w1_scale), ptr(w2), ptr(w2_scale), ptr(out),
            ptr(ws), None, m, k, n, local_experts, top_k, rank_size))
    # the launch is asynchronous: the caching allocator must not hand these blocks to another stream before it ran
    for t in (x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale, ws, out):
        t.record_stream(torch.cuda.current_stream(x.device))
    return out


_lib_def.impl("init", _init, "CompositeExplicitAutograd")
_lib_def.impl("finalize", _finalize, "CompositeExplicitAutograd")
_lib_def.impl("ascend950_dispatch_ffn_combine", _ffn, "CUDA")
_lib_def.impl("ascend950_pretile_ffn_weights", _pretile, "CUDA")
_lib_def.impl("ascend950_dispatch_ffn_combine_pretiled", _ffn_pretiled, "CUDA")
