"""Thin torch-tensor front end of the C ABI (device memory and streams only).

Every function takes CUDA(=HIP) tensors, passes raw pointers to libcatccos_mx.so on
torch's current stream and returns tensors.  bf16 data may be given as
torch.bfloat16 or as int16/uint16 bit patterns.  No function here computes
anything in torch.
"""
from __future__ import annotations

import torch

from . import _lib

FMT = {"E4M3": 0, "E5M2": 1, "E2M1": 2, "E1M2": 3}
_FP4 = ("E2M1", "E1M2")
ROUND = {"rne": 0, "lut": 1}
OUT = {"bf16": 0, "fp16": 1, "fp32": 2}
_OUT_DTYPE = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t: torch.Tensor):
    return t.data_ptr() if t is not None else None


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("expected a GPU tensor")


def scale_cols(cols: int) -> int:
    nb = (cols + 31) // 32
    return (nb + 1) // 2 * 2


def mx_quant(x: torch.Tensor, fmt: str = "E4M3", mode: str | None = None):
    """x: bf16 [rows, cols] -> (codes u8 [rows, cols or cols/2], scales u8 [rows, RoundUp2(cols/32)])."""
    _need_cuda(x)
    assert x.dim() == 2 and x.element_size() == 2 and x.stride(1) == 1
    rows, cols = x.shape
    if mode is None:
        mode = "lut" if fmt in _FP4 else "rne"
    ccols = (cols + 1) // 2 if fmt in _FP4 else cols
    codes = torch.empty((rows, ccols), dtype=torch.uint8, device=x.device)
    scales = torch.empty((rows, scale_cols(cols)), dtype=torch.uint8, device=x.device)
    lib = _lib.load()
    _lib.check(lib.cmx_mx_quant(_p(x), x.stride(0), _p(codes), ccols, _p(scales), scales.shape[1], rows, cols,
                                FMT[fmt], ROUND[mode], _stream()))
    return codes, scales


def mx_dequant(codes: torch.Tensor, scales: torch.Tensor, cols: int, fmt: str = "E4M3") -> torch.Tensor:
    _need_cuda(codes, scales)
    rows = codes.shape[0]
    out = torch.empty((rows, cols), dtype=torch.float32, device=codes.device)
    lib = _lib.load()
    _lib.check(lib.cmx_mx_dequant(_p(codes), codes.stride(0), _p(scales), scales.stride(0), _p(out), cols, rows, cols,
                                  FMT[fmt], _stream()))
    return out


def mx_gemm(a, a_scale, b, b_scale, k: int, fmt: str = "E4M3", out: str = "bf16") -> torch.Tensor:
    """C[m,n] = deq(a)[m,k] . deq(b)[n,k]^T"""
    _need_cuda(a, a_scale, b, b_scale)
    m, n = a.shape[0], b.shape[0]
    c = torch.empty((m, n), dtype=_OUT_DTYPE[out], device=a.device)
    lib = _lib.load()
    _lib.check(lib.cmx_mx_gemm(_p(a), a.stride(0), _p(a_scale), a_scale.stride(0), _p(b), b.stride(0), _p(b_scale),
                               b_scale.stride(0), _p(c), n, m, n, k, FMT[fmt], OUT[out], _stream()))
    return c


def mx_to_k_major(src, src_scale, k: int, n: int):
    """codes [batch, k, n] (or [k, n]) with scales [batch, k/64, n, 2] -> K-contiguous codes [batch, n, k], scales [batch, n, k/32]."""
    _need_cuda(src, src_scale)
    assert src.is_contiguous() and src_scale.is_contiguous()
    batch = src.shape[0] if src.dim() == 3 else 1
    shape = (batch, n) if src.dim() == 3 else (n,)
    dst = torch.empty(shape + (k,), dtype=torch.uint8, device=src.device)
    dst_scale = torch.empty(shape + (k // 32,), dtype=torch.uint8, device=src.device)
    lib = _lib.load()
    _lib.check(lib.cmx_mx_to_k_major(_p(src), n, _p(src_scale), _p(dst), k, _p(dst_scale), k // 32, k, n, batch, _stream()))
    return dst, dst_scale


def mxfp4_to_k_major(src, src_scale, k: int, n: int):
    """FP4: bytes [batch, k, ceil(n/2)] (pairs along n) with scales [batch, k/64, n, 2] -> bytes [batch, n, k/2], scales [batch, n, k/32]."""
    _need_cuda(src, src_scale)
    assert src.is_contiguous() and src_scale.is_contiguous()
    batch = src.shape[0] if src.dim() == 3 else 1
    shape = (batch, n) if src.dim() == 3 else (n,)
    dst = torch.empty(shape + (k // 2,), dtype=torch.uint8, device=src.device)
    dst_scale = torch.empty(shape + (k // 32,), dtype=torch.uint8, device=src.device)
    lib = _lib.load()
    _lib.check(lib.cmx_mxfp4_to_k_major(_p(src), (n + 1) // 2, _p(src_scale), _p(dst), k // 2, _p(dst_scale), k // 32, k, n, batch,
                                        _stream()))
    return dst, dst_scale


def mx_gemm_ex(a, a_scale, b, b_scale, m: int, n: int, k: int, fmt: str = "E4M3", out: str = "bf16", trans_a: int = 0,
               trans_b: int = 1) -> torch.Tensor:
    """Dense operands in the reference's file layouts: a [m, k] (trans_a = 1: [k, m], scales [k/64, m, 2]);
    b [n, k] (trans_b = 0: [k, n], scales [k/64, n, 2])."""
    _need_cuda(a, a_scale, b, b_scale)
    assert all(t.is_contiguous() for t in (a, a_scale, b, b_scale))
    lib = _lib.load()
    need = lib.cmx_mx_gemm_ex_workspace_bytes(m, n, k, trans_a, trans_b)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=a.device)
    c = torch.empty((m, n), dtype=_OUT_DTYPE[out], device=a.device)
    _lib.check(lib.cmx_mx_gemm_ex(_p(a), _p(a_scale), _p(b), _p(b_scale), _p(c), n, m, n, k, FMT[fmt], OUT[out], trans_a,
                                  trans_b, _p(ws), _stream()))
    return c


def mx_gmm_ex(a, a_scale, b, b_scale, group_sizes, n: int, k: int, fmt: str = "E4M3", out: str = "bf16",
              trans_b: int = 1) -> torch.Tensor:
    """Grouped form: b [G, n, k] (trans_b = 0: [G, k, n], scales [G, k/64, n, 2])."""
    _need_cuda(a, a_scale, b, b_scale, group_sizes)
    assert all(t.is_contiguous() for t in (a, a_scale, b, b_scale)) and group_sizes.dtype == torch.int32
    m, g = a.shape[0], b.shape[0]
    lib = _lib.load()
    ws = torch.empty(lib.cmx_mx_gmm_ex_workspace_bytes(g, n, k, trans_b), dtype=torch.uint8, device=a.device)
    c = torch.zeros((m, n), dtype=_OUT_DTYPE[out], device=a.device)
    _lib.check(lib.cmx_mx_gmm_ex(_p(a), _p(a_scale), _p(b), _p(b_scale), _p(c), n, _p(group_sizes), g, m, n, k, FMT[fmt],
                                 OUT[out], trans_b, _p(ws), _stream()))
    return c


def int8_quant_scatter(x: torch.Tensor, src2sorted, top_k: int = 1):
    """x bf16 [tokens, k] -> (codes int8 [tokens*top_k, k], scales fp32 [tokens*top_k]); row t goes to src2sorted[t*top_k + r]."""
    _need_cuda(x, src2sorted)
    assert x.dim() == 2 and x.element_size() == 2 and x.stride(1) == 1
    tokens, k = x.shape
    codes = torch.empty((tokens * top_k, k), dtype=torch.int8, device=x.device)
    scales = torch.empty((tokens * top_k,), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    _lib.check(lib.cmx_int8_quant_scatter(_p(x), x.stride(0), _p(src2sorted), _p(codes), k, _p(scales), tokens, k, top_k, _stream()))
    return codes, scales


def int8_gmm_dequant_swiglu(a, token_scale, b, channel_scale, group_sizes, n: int, k: int, trans_b: int = 0,
                            out: str = "fp32", scale_stride: int = 1, c=None) -> torch.Tensor:
    """a int8 [rows, k]; b int8 [G, k, n] (trans_b = 0) or [G, n, k] (trans_b = 1); channel_scale fp32 [G*n*scale_stride]."""
    _need_cuda(a, token_scale, b, channel_scale, group_sizes)
    assert a.is_contiguous() and b.is_contiguous() and group_sizes.dtype == torch.int32
    rows, g = a.shape[0], b.shape[0]
    lib = _lib.load()
    ws = torch.empty(lib.cmx_int8_gmm_workspace_bytes(g, n, k, trans_b), dtype=torch.uint8, device=a.device)
    if c is None:
        c = torch.zeros((rows, n // 2), dtype=_OUT_DTYPE[out], device=a.device)
    _lib.check(lib.cmx_int8_gmm_dequant_swiglu(_p(a), k, _p(token_scale), _p(b), _p(channel_scale), scale_stride, _p(c),
                                               c.stride(0), OUT[out], _p(group_sizes), g, rows, n, k, trans_b, _p(ws), _stream()))
    return c


def gmm_workspace(groups: int, device) -> torch.Tensor:
    lib = _lib.load()
    return torch.empty(lib.cmx_mx_gmm_workspace_bytes(groups), dtype=torch.uint8, device=device)


class PretiledWeights:
    """Expert weights [groups, n, k] (8-bit codes) in the tiled order of cmx_mx_pretile_weights; ``pair_gate_up``
    says which of the two grouped matmuls the tiling is for (True: mx_gmm_swiglu_quant, False: mx_gmm)."""

    def __init__(self, data: torch.Tensor, groups: int, n: int, k: int, pair_gate_up: bool):
        self.data, self.groups, self.n, self.k, self.pair_gate_up = data, groups, n, k, pair_gate_up

    @property
    def shape(self):
        return (self.groups, self.n, self.k)


def pretile_weights(b: torch.Tensor, pair_gate_up: bool) -> PretiledWeights:
    """b u8 [G, n, k] dense -> PretiledWeights (one pass over the weights; meant for weight-load time)."""
    _need_cuda(b)
    assert b.dtype == torch.uint8 and b.dim() == 3 and b.is_contiguous()
    g, n, k = b.shape
    lib = _lib.load()
    nbytes = lib.cmx_mx_pretiled_weight_bytes(g, n, k, int(pair_gate_up))
    if nbytes == 0:
        raise ValueError("pre-tiled weights need k % 512 == 0 (and n % 64 == 0 for gate|up weights)")
    out = torch.empty(nbytes, dtype=torch.uint8, device=b.device)
    _lib.check(lib.cmx_mx_pretile_weights(_p(b), _p(out), g, n, k, int(pair_gate_up), _stream()))
    return PretiledWeights(out, g, n, k, bool(pair_gate_up))


def _weights(b, pair_gate_up: bool):
    """(pointer, pretiled?) of a weight argument: a dense tensor or PretiledWeights of the matching kind."""
    if isinstance(b, PretiledWeights):
        assert b.pair_gate_up == pair_gate_up, "weights were pre-tiled for the other grouped matmul"
        return _p(b.data), True
    assert b.is_contiguous()
    return _p(b), False


def mx_gmm(a, a_scale, b, b_scale, group_sizes, k: int, fmt: str = "E4M3", out: str = "bf16", c=None, workspace=None):
    """a [m_total, k], b [G, n, k] (dense tensor or PretiledWeights), group_sizes int32 [G] on device -> c [m_total, n]
    (rows past the groups untouched)."""
    _need_cuda(a, a_scale, b_scale, group_sizes)
    assert b_scale.is_contiguous() and group_sizes.dtype == torch.int32
    bp, tiled = _weights(b, False)
    m, (g, n) = a.shape[0], b.shape[:2]
    if c is None:
        c = torch.zeros((m, n), dtype=_OUT_DTYPE[out], device=a.device)
    if workspace is None:
        workspace = gmm_workspace(g, a.device)
    lib = _lib.load()
    fn = lib.cmx_mx_gmm_pretiled if tiled else lib.cmx_mx_gmm
    _lib.check(fn(_p(a), a.stride(0), _p(a_scale), a_scale.stride(0), bp, _p(b_scale), _p(c), c.stride(0),
                  _p(group_sizes), g, m, n, k, FMT[fmt], OUT[out], _p(workspace), _stream()))
    return c


def mx_gmm_swiglu_quant(a, a_scale, b, b_scale, group_sizes, k: int, want_bf16: bool = False, workspace=None,
                        outs=None):
    """GMM1 + SwiGLU + MX requant.  b [G, n, k] (gate rows then up rows; dense tensor or PretiledWeights).
    Returns (codes [m, n/2], scales, act_bf16|None)."""
    _need_cuda(a, a_scale, b_scale, group_sizes)
    assert b_scale.is_contiguous() and group_sizes.dtype == torch.int32
    bp, tiled = _weights(b, True)
    m, (g, n) = a.shape[0], b.shape[:2]
    half = n // 2
    if outs is None:
        codes = torch.zeros((m, half), dtype=torch.uint8, device=a.device)
        scales = torch.zeros((m, scale_cols(half)), dtype=torch.uint8, device=a.device)
    else:
        codes, scales = outs
    act = torch.zeros((m, half), dtype=torch.bfloat16, device=a.device) if want_bf16 else None
    if workspace is None:
        workspace = gmm_workspace(g, a.device)
    lib = _lib.load()
    fn = lib.cmx_mx_gmm_swiglu_quant_pretiled if tiled else lib.cmx_mx_gmm_swiglu_quant
    _lib.check(fn(_p(a), a.stride(0), _p(a_scale), a_scale.stride(0), bp, _p(b_scale), _p(codes), codes.stride(0),
                  _p(scales), scales.stride(0), _p(act), _p(group_sizes), g, m, n, k, _p(workspace), _stream()))
    return codes, scales, act


def mx_gmm_swiglu_quant_noalloc(a, a_scale, b, b_scale, group_sizes, k: int, codes, scales, act=None) -> None:
    """cmx_mx_gmm_swiglu_quant_noalloc: the caller brings every buffer (codes [m, n/2], scales, optional bf16 act);
    neither this wrapper nor the library allocates anything."""
    _need_cuda(a, a_scale, b, b_scale, group_sizes, codes, scales)
    assert b.is_contiguous() and b_scale.is_contiguous() and group_sizes.dtype == torch.int32
    m, (g, n) = a.shape[0], b.shape[:2]
    lib = _lib.load()
    _lib.check(lib.cmx_mx_gmm_swiglu_quant_noalloc(_p(a), a.stride(0), _p(a_scale), a_scale.stride(0), _p(b), _p(b_scale),
                                                   _p(codes), codes.stride(0), _p(scales), scales.stride(0), _p(act),
                                                   _p(group_sizes), g, m, n, k, _stream()))


def init() -> None:
    """cmx_init on the current device."""
    _lib.check(_lib.load().cmx_init())


def moe_init_routing(expert_idx: torch.Tensor, experts: int):
    """expert_idx int32 [T, topK] -> (sorted2src, src2sorted, counts) int32."""
    _need_cuda(expert_idx)
    assert expert_idx.dtype == torch.int32 and expert_idx.is_contiguous()
    t, top_k = expert_idx.shape
    dev = expert_idx.device
    s2s = torch.empty(t * top_k, dtype=torch.int32, device=dev)
    inv = torch.empty(t * top_k, dtype=torch.int32, device=dev)
    counts = torch.empty(experts, dtype=torch.int32, device=dev)
    lib = _lib.load()
    ws = torch.empty(lib.cmx_moe_routing_workspace_bytes(t * top_k, experts), dtype=torch.uint8, device=dev)
    _lib.check(lib.cmx_moe_init_routing(_p(expert_idx), t, top_k, experts, _p(s2s), _p(inv), _p(counts), _p(ws),
                                        _stream()))
    return s2s, inv, counts


def quant_scatter(x: torch.Tensor, src2sorted: torch.Tensor, top_k: int, packed: bool = False, out=None):
    """x bf16 [T, k] -> rows quantised once and written to their top_k destinations.
    packed=False: (codes [T*topK, k], scales [T*topK, RoundUp2(k/32)]);
    packed=True: one buffer [T*topK, packed_row_bytes(k)] = codes | scales | pad (``out``: a caller's zeroed buffer
    of that shape)."""
    _need_cuda(x, src2sorted)
    t, k = x.shape
    rows = t * top_k
    lib = _lib.load()
    if packed:
        rb = lib.cmx_packed_row_bytes(k)
        buf = torch.zeros((rows, rb), dtype=torch.uint8, device=x.device) if out is None else out
        assert buf.shape == (rows, rb) and buf.dtype == torch.uint8 and buf.is_contiguous()
        _lib.check(lib.cmx_quant_scatter(_p(x), x.stride(0), _p(src2sorted), _p(buf), rb, buf.data_ptr() + k, rb, t, k,
                                         top_k, _stream()))
        return buf
    codes = torch.zeros((rows, k), dtype=torch.uint8, device=x.device)
    scales = torch.zeros((rows, scale_cols(k)), dtype=torch.uint8, device=x.device)
    _lib.check(lib.cmx_quant_scatter(_p(x), x.stride(0), _p(src2sorted), _p(codes), k, _p(scales), scales.shape[1], t, k,
                                     top_k, _stream()))
    return codes, scales


def moe_token_unpermute(y: torch.Tensor, src2sorted: torch.Tensor, probs: torch.Tensor) -> torch.Tensor:
    """y bf16 [rows, h]; probs fp32 [T, topK] -> bf16 [T, h]."""
    _need_cuda(y, src2sorted, probs)
    assert probs.dtype == torch.float32 and probs.is_contiguous()
    t, top_k = probs.shape
    rows, h = y.shape
    out = torch.empty((t, h), dtype=y.dtype, device=y.device)
    lib = _lib.load()
    _lib.check(lib.cmx_moe_token_unpermute(_p(y), y.stride(0), rows, _p(src2sorted), _p(probs), _p(out), h, t, h, top_k,
                                           _stream()))
    return out


def ffn_workspace_bytes(m: int, k: int, n: int, experts: int, top_k: int) -> int:
    return _lib.load().catccos_ascend950_dispatch_ffn_combine_workspace_bytes(m, k, n, experts, top_k, 1)


def ffn_workspace_layout(m: int, k: int, n: int, experts: int, top_k: int) -> dict:
    lay = _lib.FfnWorkspaceLayout()
    _lib.check(_lib.load().cmx_ffn_workspace_layout_get(m, k, n, experts, top_k, lay))
    return {f: getattr(lay, f) for f, _ in lay._fields_}


def dispatch_ffn_combine(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale, workspace=None, out=None):
    """torch.ops.catccos.ascend950_dispatch_ffn_combine(x, expert_idx, gate_weight, w1, w1_scale, w2, w2_scale)
    on one GPU: x bf16 [m,k]; expert_idx int32 [m,topK]; gate_weight fp32 [m,topK];
    w1 [E,n,k] + w1_scale [E,n,k/32]; w2 [E,k,n/2] + w2_scale [E,k,n/64] -> bf16 [m,k].
    w1 and w2 may both be PretiledWeights (w1 tiled with pair_gate_up=True, w2 with False): same result, through
    cmx_dispatch_ffn_combine_pretiled."""
    _need_cuda(x, expert_idx, gate_weight, w1_scale, w2_scale)
    m, k = x.shape
    e, n = w1.shape[:2]
    top_k = expert_idx.shape[1]
    for t in (x, expert_idx, gate_weight, w1_scale, w2_scale):
        assert t.is_contiguous()
    w1p, tiled1 = _weights(w1, True)
    w2p, tiled2 = _weights(w2, False)
    assert tiled1 == tiled2, "pre-tile both weight tensors or neither"
    lib = _lib.load()
    if workspace is None:
        workspace = torch.empty(ffn_workspace_bytes(m, k, n, e, top_k), dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((m, k), dtype=x.dtype, device=x.device)
    if tiled1:
        _lib.check(lib.cmx_dispatch_ffn_combine_pretiled(
            _stream(), _p(x), _p(expert_idx), _p(gate_weight), w1p, _p(w1_scale), w2p, _p(w2_scale), _p(out),
            _p(workspace), m, k, n, e, top_k))
        return out
    _lib.check(lib.catccos_ascend950_dispatch_ffn_combine(
        0, _stream(), 0, _p(x), _p(expert_idx), _p(gate_weight), w1p, _p(w1_scale), w2p, _p(w2_scale), _p(out),
        _p(workspace), None, m, k, n, e, top_k, 1))
    return out
