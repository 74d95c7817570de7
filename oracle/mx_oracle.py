"""CPU oracle for the MX compute core (TEST INFRASTRUCTURE - never on the product path).

This module restates, in plain numpy, the arithmetic that the reference's Python
golden generators define for MX block quantization, MX matmul / grouped matmul,
SwiGLU + requant, MoE routing and the weighted top-k combine.  Only tests, the
smoke check and the CPU-baseline leg of the benchmark may import it; the shipped
library never does.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  Bit-level conventions:

* bf16 tensors travel as ``uint16`` bit patterns, FP8/FP4/E8M0 as ``uint8``.
* "RNE" = IEEE round-to-nearest-even; "LUT" = nearest table value with ties to
  the smaller magnitude and -0 canonicalised to +0 (first-index arg-min).

Pinning status (see tests/test_oracle_*.py, tests/test_golden_fixtures.py): E8M0 exponent,
E4M3/E5M2 RNE (vs the torch CPU cast and brute force over all bf16 patterns), E4M3/E2M1
LUT (vs the 256-/16-entry arg-min definition), FP4 packing, bf16 RNE, routing, combine,
workspace sizing (literal hand-computed sums) and both acceptance rules (literal cases at
and one step beyond every threshold) are pinned.  The quantizers (every format and
rounding, ties, signed zeros, tiny / all-zero blocks, Inf and NaN) and the whole FFN chain
are also pinned bit for bit by vectors that the reference's own Python goldens produced
(tests/golden/*.npz, made by tests/golden/make_fixtures.py).  MX GEMM results of the
reference DEVICE are pinned only through tolerance and special cases (the bit-level
accumulate order of its matmul lives in an absent third-party library): exact device GEMM
bits are "parity unpinned".
"""
from __future__ import annotations

import numpy as np

BLOCK = 32          # gen_mx_quant_allgather_data.py:22  (_BLOCK_SIZE)
EPSILON = 1e-12     # gen_mx_quant_allgather_data.py:23
E8M0_BIAS = 127

# element formats: name -> (emax, max_value)   gen_mx_quant_allgather_data.py:41-73
FORMATS = {
    "E4M3": dict(emax=8, max_value=448.0),
    "E5M2": dict(emax=15, max_value=57344.0),
    "E2M1": dict(emax=2, max_value=6.0),
    "E1M2": dict(emax=0, max_value=1.75),
}


# --------------------------------------------------------------------------- #
# bf16 helpers                                      examples/utils/utils.py:64-94
# --------------------------------------------------------------------------- #
def f32_to_bf16_bits(x) -> np.ndarray:
    """fp32 -> bf16 bit pattern, round-to-nearest-even (``bits += 0x7FFF + lsb``,
    utils.py:85-87).  NaN maps to a quiet NaN; the sign of zero is kept, as the
    torch cast used by the golden path (gen_data_moe.py:650) keeps it."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    out = rounded.astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), out)
    return out.reshape(x.shape)


def bf16_bits_to_f32(b) -> np.ndarray:
    """bf16 bit pattern -> fp32 (exact).  utils.py:92-94"""
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def bf16_round(x) -> np.ndarray:
    """fp32 -> nearest bf16, returned as fp32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


# --------------------------------------------------------------------------- #
# decode tables
# --------------------------------------------------------------------------- #
def e4m3_table() -> np.ndarray:
    """256-entry E4M3 (fn) value table as the reference builds it
    (gen_mx_quant_allgather_data.py:79-102): index 127/255 hold +-448 rather than
    NaN, index 128 is -0."""
    v = np.zeros(256, dtype=np.float32)
    for i in range(256):
        sign = 1.0 if i < 128 else -1.0
        m = i & 0x7F
        if m == 0:
            val = 0.0
        elif m == 127:
            val = 448.0
        else:
            e, f = (m >> 3) & 0xF, m & 7
            val = (f / 8.0) * 2.0 ** (1 - 7) if e == 0 else (1 + f / 8.0) * 2.0 ** (e - 7)
        v[i] = sign * min(val, 448.0)
    return v


def e5m2_table() -> np.ndarray:
    """gen_mx_quant_allgather_data.py:105-128 (indices 124..127 clamp to 57344)."""
    v = np.zeros(256, dtype=np.float32)
    for i in range(256):
        sign = 1.0 if i < 128 else -1.0
        m = i & 0x7F
        if m == 0:
            val = 0.0
        elif m >= 124:
            val = 57344.0
        else:
            e, f = (m >> 2) & 0x1F, m & 3
            val = (f / 4.0) * 2.0 ** (1 - 15) if e == 0 else (1 + f / 4.0) * 2.0 ** (e - 15)
        v[i] = sign * min(val, 57344.0)
    return v


def fp4_table(fmt: str = "E2M1") -> np.ndarray:
    """16-entry FP4 table, sign in bit 3.  gen_mx_quant_allgather_data.py:352-376"""
    exp_bits, man_bits, bias = (2, 1, 1) if fmt == "E2M1" else (1, 2, 1)
    v = np.zeros(16, dtype=np.float32)
    for i in range(16):
        s = (i >> 3) & 1
        e = (i >> man_bits) & ((1 << exp_bits) - 1)
        f = i & ((1 << man_bits) - 1)
        if e == 0:
            val = (f / float(1 << man_bits)) * 2.0 ** (1 - bias)
        else:
            val = (1 + f / float(1 << man_bits)) * 2.0 ** (e - bias)
        v[i] = -val if s else val
    return v


_E4M3 = e4m3_table()
_E5M2 = e5m2_table()
_FP4 = {"E2M1": fp4_table("E2M1"), "E1M2": fp4_table("E1M2")}
_FP8 = {"E4M3": _E4M3, "E5M2": _E5M2}


def decode(codes, fmt: str) -> np.ndarray:
    """Element code -> fp32 value (FP4 codes are one nibble per array entry)."""
    codes = np.asarray(codes)
    if fmt in _FP8:
        return _FP8[fmt][codes.astype(np.uint8)]
    return _FP4[fmt][codes.astype(np.uint8) & 0xF]


# --------------------------------------------------------------------------- #
# E8M0 shared exponent              gen_mx_quant_allgather_data.py:168-189
# --------------------------------------------------------------------------- #
def e8m0_exp(amax, emax: int) -> np.ndarray:
    """``0 if amax < 1e-12 else clamp(floor(log2 amax) - emax, -128, 127)`` with
    floor(log2) read from the fp32 exponent field (:181-189)."""
    amax = np.ascontiguousarray(amax, dtype=np.float32)
    zero = amax < np.float32(EPSILON)
    safe = np.where(zero, np.float32(1.0), amax)
    bits = safe.view(np.uint32).astype(np.int64)
    e = ((bits >> 23) & 0xFF) - 127 - emax
    e = np.clip(e, -128, 127)
    return np.where(zero, 0, e).astype(np.int32)


def e8m0_byte(exp) -> np.ndarray:
    """Stored byte = exponent + 127 (torch.exp2(e).to(float8_e8m0fnu), :282,341).
    exponent -128 has no E8M0 encoding below byte 0; it saturates to byte 0."""
    return np.clip(np.asarray(exp, dtype=np.int32) + E8M0_BIAS, 0, 254).astype(np.uint8)


# --------------------------------------------------------------------------- #
# element encoders
# --------------------------------------------------------------------------- #
def _fp8_rne(y, man_bits: int, bias: int, max_code: int) -> np.ndarray:
    """IEEE RNE of a finite fp32 (already clamped to the format's range) to an
    8-bit float with ``man_bits`` mantissa bits; sign kept on underflow (the torch
    cast behind the 'native' backend, gen_mx_quant_allgather_data.py:291-292)."""
    y = np.ascontiguousarray(y, dtype=np.float32)
    bits = y.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    a = (bits & 0x7FFFFFFF).astype(np.int64)
    drop = 23 - man_bits
    # normal numbers: round the mantissa, let the carry ripple into the exponent
    rounded = a + ((1 << (drop - 1)) - 1) + ((a >> drop) & 1)
    code_n = (rounded >> drop) - ((127 - bias) << man_bits)
    # subnormals: value = k * 2^(1-bias-man_bits), k = RNE(|y| / step)
    step_log2 = 1 - bias - man_bits
    mag = np.where(np.isnan(y), 0.0, np.abs(y).astype(np.float64))       # NaN is patched in below
    code_s = np.rint(mag * 2.0 ** (-step_log2)).astype(np.int64)
    min_normal = 2.0 ** (1 - bias)
    code = np.where(mag < min_normal, code_s, code_n)
    code = np.minimum(code, max_code)
    out = code.astype(np.uint8) | sign
    nan = np.isnan(y)
    if nan.any():
        out = np.where(nan, sign | 0x7F, out)
    return out.reshape(y.shape)


def e4m3_encode_rne(y) -> np.ndarray:
    return _fp8_rne(y, 3, 7, 0x7E)


def e5m2_encode_rne(y) -> np.ndarray:
    return _fp8_rne(y, 2, 15, 0x7B)


def _lut_pos_encode(y, pos: np.ndarray) -> np.ndarray:
    """Vectorised arg-min on the ascending positive half of a value table, ties
    to the lower neighbour, -0 -> +0.  gen_mx_quant_allgather_data.py:198-247"""
    y = np.ascontiguousarray(y, dtype=np.float32)
    mag = np.abs(y)
    last = pos.size - 1
    upper = np.minimum(np.searchsorted(pos, mag, side="left"), last)
    lower = np.maximum(upper - 1, 0)
    uv, lv = pos[upper], pos[lower]
    pick_lower = (mag - lv) <= (uv - mag)
    idx = np.where(pick_lower, lower, upper)
    neg = (y < 0) & (pos[idx] != 0)
    return idx.astype(np.uint8), neg


def fp8_encode_lut(y, fmt: str = "E4M3") -> np.ndarray:
    """Table-search encode.  A NaN element comes out as code 0: the golden's torch.searchsorted puts NaN at
    index 0, whose table value 0 is then canonicalised to +0 (pinned by the reference-made vectors)."""
    y = np.ascontiguousarray(y, dtype=np.float32)
    nan = np.isnan(y)
    idx, neg = _lut_pos_encode(np.where(nan, np.float32(0), y), _FP8[fmt][:128])
    return (idx | np.where(neg, 0x80, 0).astype(np.uint8)).astype(np.uint8)


def fp8_encode_lut_argmin(y, fmt: str = "E4M3") -> np.ndarray:
    """Definition form: arg-min over the full 256-entry table, lowest index wins
    (legacy per-element loop, gen_data_fp8_mx_allgather_matmul.py:218-244).  The
    table is scanned in index order with a strict '<' so the first minimum wins;
    O(256 n) but needs no (n, 256) temporary."""
    tab = _FP8[fmt]
    y = np.ascontiguousarray(y, dtype=np.float32).ravel()
    best = np.abs(tab[0] - y)
    idx = np.zeros(y.shape, dtype=np.uint8)
    for i in range(1, 256):
        d = np.abs(tab[i] - y)
        better = d < best
        best = np.where(better, d, best)
        idx = np.where(better, np.uint8(i), idx)
    return idx


def fp4_encode_lut(y, fmt: str = "E2M1") -> np.ndarray:
    """Arg-min over the 16-entry table in index order, first index wins => tie to
    the smaller magnitude, -0 -> code 0.  gen_mx_quant_allgather_data.py:385-397"""
    tab = _FP4[fmt]
    y = np.ascontiguousarray(y, dtype=np.float32)
    best = np.abs(tab[0] - y)
    idx = np.zeros(y.shape, dtype=np.uint8)
    for i in range(1, 16):
        d = np.abs(tab[i] - y)
        better = d < best
        best = np.where(better, d, best)
        idx = np.where(better, np.uint8(i), idx)
    return idx


def fp4_encode_rne(y, fmt: str = "E2M1") -> np.ndarray:
    """Round-to-nearest-even onto the FP4 grid (the device quantizer's CAST_RINT,
    comm_block_mx_quant.hpp:538-555); ties go to the code with an even mantissa
    bit.  Sign is kept on underflow."""
    tab = _FP4[fmt][:8]
    y = np.ascontiguousarray(y, dtype=np.float32)
    mag = np.abs(y).astype(np.float64)
    code = np.zeros(y.shape, dtype=np.int64)
    for i in range(7):
        mid = (float(tab[i]) + float(tab[i + 1])) / 2
        up = (mag > mid) | ((mag == mid) & (((i + 1) & 1) == 0))
        code = np.where(up, i + 1, code)
    # a NaN (only reachable in a block whose maximum is NaN) encodes as +0, like the table search
    return np.where(np.isnan(y), 0, code | np.where(np.signbit(y), 8, 0)).astype(np.uint8)


def pack_fp4(codes) -> np.ndarray:
    """Two codes per byte, even column in the low nibble; an odd trailing column
    is padded with code 0.  gen_mx_quant_allgather_data.py:400-411"""
    codes = np.asarray(codes, dtype=np.uint8)
    if codes.shape[-1] % 2:
        pad = np.zeros(codes.shape[:-1] + (1,), dtype=np.uint8)
        codes = np.concatenate([codes, pad], axis=-1)
    return (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)


def unpack_fp4(packed) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = packed & 0xF
    out[..., 1::2] = packed >> 4
    return out


# --------------------------------------------------------------------------- #
# MX block quantizer
# --------------------------------------------------------------------------- #
def scale_cols(n: int) -> int:
    """Scale bytes per row: ceil(n/32) rounded up to an even count
    (gen_mx_quant_allgather_data.py:306-311; ascend950_dispatch_ffn_combine_host.h:32-33)."""
    nb = (n + BLOCK - 1) // BLOCK
    return (nb + 1) // 2 * 2


def mx_quant(x, fmt: str = "E4M3", mode: str | None = None):
    """MX-quantize fp32 ``x`` [M, N] along the last axis in blocks of 32.

    Returns ``(codes, scales)``: codes uint8 [M, N] (FP4: one nibble per entry,
    un-packed; use :func:`pack_fp4`), scales uint8 [M, scale_cols(N)] (padding
    columns hold byte 127 = 1.0).

    fmt in E4M3/E5M2 follows ``_quantize_axis_last_fp8``
    (gen_mx_quant_allgather_data.py:255-313): amax -> E8M0 exponent -> divide ->
    clamp to +-max -> cast.  mode 'rne' is the 'native' backend / the runtime
    activation quantizer ``dynamic_quant_rne`` (gen_data_moe.py:574-585); mode
    'lut' is the default offline backend.  fmt in E2M1/E1M2 follows
    ``_quantize_axis_last`` (:414-449); mode 'lut' is the golden, 'rne' the
    device rounding.  Default mode: 'rne' for FP8, 'lut' for FP4.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, n = x.shape
    f = FORMATS[fmt]
    if mode is None:
        mode = "rne" if fmt in _FP8 else "lut"
    nb = (n + BLOCK - 1) // BLOCK
    pn = nb * BLOCK
    if pn != n:
        xp = np.zeros((m, pn), dtype=np.float32)
        xp[:, :n] = x
    else:
        xp = x
    blocks = xp.reshape(m, nb, BLOCK)
    with np.errstate(invalid="ignore"):
        amax = np.abs(blocks).max(axis=-1)                  # NaN if the block holds one
    exp = e8m0_exp(amax, f["emax"])
    nan_block = np.zeros(amax.shape, dtype=bool)
    if fmt not in _FP8:
        # the FP4 golden takes floor(log2(amax)) in floating point (:429-432): an Inf maximum gives the largest
        # exponent, a NaN maximum a NaN scale (byte 255) and with it NaN quotients, which the table search
        # sends to code 0
        exp = np.where(np.isinf(amax), 127, exp).astype(np.int32)
        nan_block = np.isnan(amax)
    # division by an exact power of two == scaling by 2^-exp (ldexp is exact)
    with np.errstate(invalid="ignore", over="ignore"):
        scaled = np.ldexp(blocks, -exp[..., None]).astype(np.float32)
    mv = np.float32(f["max_value"])
    scaled = np.clip(scaled, -mv, mv)                       # NaN stays NaN, as torch.clamp leaves it
    scaled = np.where(nan_block[..., None], np.float32(np.nan), scaled)
    if fmt == "E4M3":
        codes = e4m3_encode_rne(scaled) if mode == "rne" else fp8_encode_lut(scaled, "E4M3")
    elif fmt == "E5M2":
        codes = e5m2_encode_rne(scaled) if mode == "rne" else fp8_encode_lut(scaled, "E5M2")
    else:
        codes = fp4_encode_rne(scaled, fmt) if mode == "rne" else fp4_encode_lut(scaled, fmt)
    codes = codes.reshape(m, pn)[:, :n]
    sc = np.full((m, scale_cols(n)), E8M0_BIAS, dtype=np.uint8)
    sc[:, :nb] = np.where(nan_block, np.uint8(255), e8m0_byte(exp))
    return np.ascontiguousarray(codes), sc


def mx_dequant(codes, scales, fmt: str = "E4M3") -> np.ndarray:
    """``value(code) * 2^(byte-127)`` per block of 32 along the last axis
    (gen_mx_quant_allgather_data.py:299; gen_data_mxfp8_mmrs.py:349-352)."""
    codes = np.asarray(codes)
    m, n = codes.shape
    nb = (n + BLOCK - 1) // BLOCK
    vals = decode(codes, fmt)
    e = np.asarray(scales)[:, :nb].astype(np.int32) - E8M0_BIAS
    e = np.repeat(e, BLOCK, axis=1)[:, :n]
    return np.ldexp(vals, e).astype(np.float32)


def mx_quant_bf16(x_bits, fmt: str = "E4M3", mode: str | None = None):
    """Quantizer entry for bf16 bit patterns (what the operator reads)."""
    return mx_quant(bf16_bits_to_f32(x_bits), fmt, mode)


# --------------------------------------------------------------------------- #
# MX GEMM / grouped GEMM
# --------------------------------------------------------------------------- #
def mx_gemm_f32(a_codes, a_scales, b_codes, b_scales, fmt_a="E4M3", fmt_b="E4M3") -> np.ndarray:
    """fp32 high-precision golden: deq(A)[M,K] @ deq(B)[N,K]^T, both operands
    K-contiguous (transposed weights, gen_data_moe.py:639-651;
    gen_data_mxfp8_mmrs.py:343-345)."""
    a = mx_dequant(a_codes, a_scales, fmt_a)
    b = mx_dequant(b_codes, b_scales, fmt_b)
    return a @ b.T


def to_file_layout(codes, scales, trans: bool):
    """K-contiguous operand (codes [R, K], scales [R, K/32]) -> the reference's file layout.
    trans False ("stored transposed", B with trans_b = 1 / A with trans_a = 0): codes [R, K], scales
    [R, K/64, 2] -- the same bytes.  trans True (B with trans_b = 0 / A with trans_a = 1): codes [K, R],
    scales [K/64, R, 2].  gen_data_mxfp8_mmrs.py:311-330 (reshape to pairs, then permute(0, 2, 1) resp.
    permute(1, 0, 2))."""
    codes = np.asarray(codes)
    scales = np.asarray(scales)
    r, k = codes.shape
    pairs = scales[:, :k // 32].reshape(r, k // 64, 2)
    if not trans:
        return np.ascontiguousarray(codes), np.ascontiguousarray(pairs)
    return np.ascontiguousarray(codes.T), np.ascontiguousarray(pairs.transpose(1, 0, 2))


def from_file_layout(codes, scales, trans: bool):
    """Inverse of :func:`to_file_layout`: back to codes [R, K], scales [R, K/32]."""
    codes = np.asarray(codes)
    scales = np.asarray(scales)
    if not trans:
        r, k = codes.shape
        return np.ascontiguousarray(codes), np.ascontiguousarray(scales.reshape(r, k // 32))
    k, r = codes.shape
    return np.ascontiguousarray(codes.T), np.ascontiguousarray(scales.reshape(k // 64, r, 2).transpose(1, 0, 2).reshape(r, k // 32))


def to_file_layout_fp4(codes, scales, trans: bool):
    """FP4 counterpart of :func:`to_file_layout` for un-packed codes [R, K]: the generator packs two codes per byte
    along the LAST axis of whichever orientation it writes (matrix_fp32_to_fp4,
    gen_data_fp4_mx_alltoallv_gmm.py:522-545; orientation and scale permutes :586-620).  trans False: bytes
    [R, K/2] (pairs along K), scales [R, K/64, 2].  trans True: bytes [K, ceil(R/2)] (pairs along R), scales
    [K/64, R, 2]."""
    codes = np.asarray(codes)
    scales = np.asarray(scales)
    r, k = codes.shape
    pairs = scales[:, :k // 32].reshape(r, k // 64, 2)
    if not trans:
        return pack_fp4(codes), np.ascontiguousarray(pairs)
    return pack_fp4(np.ascontiguousarray(codes.T)), np.ascontiguousarray(pairs.transpose(1, 0, 2))


def group_offsets(counts) -> np.ndarray:
    """Exclusive prefix of rows per expert (EP = 1 case of
    PrepareDstExpertOffsets, ascend950_dispatch_ffn_combine_device.h:406-441)."""
    counts = np.asarray(counts, dtype=np.int64)
    off = np.zeros(counts.size + 1, dtype=np.int64)
    np.cumsum(counts, out=off[1:])
    return off


def cumsum_for_mm(tokens_per_expert, rank: int, ep: int, epr: int) -> np.ndarray:
    """Inclusive prefix over source ranks of this rank's local-expert columns of
    the [EP, EP*epr] tokens-per-expert table
    (comm_block_scheduler_alltoallv_gmm.hpp:123-156).  Row EP-1 holds the group
    sizes the matmul loop reads (ascend950_alltoall_gmm.hpp:240)."""
    t = np.asarray(tokens_per_expert, dtype=np.int32).reshape(ep, ep * epr)
    return np.cumsum(t[:, rank * epr:(rank + 1) * epr], axis=0, dtype=np.int32)


def src_prev_sum(tokens_per_expert, core_idx: int, rank: int, ep: int, epr: int) -> int:
    """Rows of source rank ``core_idx`` routed to experts of lower ranks
    (SetCommCore, comm_block_scheduler_alltoallv_gmm.hpp:101-113)."""
    t = np.asarray(tokens_per_expert, dtype=np.int64).ravel()
    if core_idx >= ep:
        return 0
    base = core_idx * ep * epr
    return int(t[base:base + rank * epr].sum())


def mx_gmm_f32(a_codes, a_scales, b_codes, b_scales, counts, fmt_a="E4M3", fmt_b="E4M3"):
    """Grouped matmul: rows [off[g], off[g+1]) of A times expert g's weight
    B[g] [N, K] (gen_data_moe.py:646-651; gen_data_fp4_mx_alltoallv_gmm.py:724-734)."""
    off = group_offsets(counts)
    n = b_codes.shape[1]
    out = np.zeros((a_codes.shape[0], n), dtype=np.float32)
    for g in range(len(counts)):
        lo, hi = int(off[g]), int(off[g + 1])
        if hi > lo:
            out[lo:hi] = mx_gemm_f32(a_codes[lo:hi], a_scales[lo:hi], b_codes[g], b_scales[g], fmt_a, fmt_b)
    return out


def swiglu_bf16(h_bits) -> np.ndarray:
    """bf16( silu_fp32(h[:, :N/2]) * h[:, N/2:] ) on bf16 input (bit patterns).
    gen_data_moe.py:655-656: ``act * sigmoid(act) * gate`` evaluated in fp32."""
    h = bf16_bits_to_f32(h_bits)
    half = h.shape[1] // 2
    act, up = h[:, :half], h[:, half:]
    with np.errstate(over="ignore"):      # exp(-act) = inf for act < -88.7 gives sigmoid 0, the fp32 result
        sig = (np.float32(1.0) / (np.float32(1.0) + np.exp(-act, dtype=np.float32))).astype(np.float32)
    return f32_to_bf16_bits((act * sig).astype(np.float32) * up)


def gmm1_swiglu_quant(a_codes, a_scales, w1_codes, w1_scales, counts):
    """GMM1 -> bf16 -> SwiGLU -> bf16 -> MX requant (RNE).  gen_data_moe.py:646-658.
    Returns (h_bf16_bits [M, N], act_bf16_bits [M, N/2], codes [M, N/2], scales)."""
    h = f32_to_bf16_bits(mx_gmm_f32(a_codes, a_scales, w1_codes, w1_scales, counts))
    act = swiglu_bf16(h)
    q, s = mx_quant_bf16(act, "E4M3", "rne")
    return h, act, q, s


# --------------------------------------------------------------------------- #
# routing / combine
# --------------------------------------------------------------------------- #
def moe_init_routing(expert_idx, expert_num: int):
    """Stable sort of the flattened [T, topK] expert ids.
    gen_data_moe.py:48-57 (sorted2src = argsort(stable), counts = bincount) and the
    device's inverse index src2sorted[sorted2src[i]] = i
    (moe_v2_src_to_dst_op_simt.h:79-87).  Returns int32 arrays."""
    flat = np.asarray(expert_idx).reshape(-1).astype(np.int64)
    sorted2src = np.argsort(flat, kind="stable").astype(np.int32)
    counts = np.bincount(flat, minlength=expert_num).astype(np.int32)
    src2sorted = np.empty_like(sorted2src)
    src2sorted[sorted2src] = np.arange(flat.size, dtype=np.int32)
    return sorted2src, src2sorted, counts


def packed_row_bytes(k: int) -> int:
    """[codes K | scales RoundUp2(K/32) | pad to 32 B]
    (comm_block_mx_quant.hpp:326-330)."""
    return (k + scale_cols(k) + 31) // 32 * 32


def quant_scatter_packed(x_bits, src2sorted, top_k: int):
    """Quantize every token once (E4M3, RNE) and write its packed row to each of
    its topK destinations src2sorted[t*topK + r]; negative destinations are
    skipped (comm_block_mx_quant.hpp:318-368).  Returns uint8 [T*topK, rowBytes]
    (pad bytes zero)."""
    x_bits = np.asarray(x_bits, dtype=np.uint16)
    t, k = x_bits.shape
    q, s = mx_quant_bf16(x_bits, "E4M3", "rne")
    rb = packed_row_bytes(k)
    out = np.zeros((t * top_k, rb), dtype=np.uint8)
    dst = np.asarray(src2sorted, dtype=np.int64).reshape(t, top_k)
    for r in range(top_k):
        ok = dst[:, r] >= 0
        out[dst[ok, r], :k] = q[ok]
        out[dst[ok, r], k:k + s.shape[1]] = s[ok]
    return out


def unpermute_combine(y_bits, src2sorted, probs) -> np.ndarray:
    """out[t] = sum_k probs[t,k] * y[src2sorted[t*topK+k]]: fp32 multiply then
    fp32 add, in k order, then RNE to bf16 (moe_token_unpermute.h:233-276,
    :296-349: Muls then Add, CAST_RINT on output).  Rows whose index is
    >= the number of permuted rows contribute nothing (:245-254)."""
    y = bf16_bits_to_f32(y_bits)
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    t, top_k = probs.shape
    idx = np.asarray(src2sorted, dtype=np.int64).reshape(t, top_k)
    acc = np.zeros((t, y.shape[1]), dtype=np.float32)
    nrows = y.shape[0]
    for k in range(top_k):
        ok = (idx[:, k] < nrows) & (idx[:, k] >= 0)
        rows = np.where(ok, idx[:, k], 0)
        term = (y[rows] * probs[:, k:k + 1]).astype(np.float32)
        term[~ok] = 0.0
        if k == 0:
            acc = term
        else:
            acc = (acc + term).astype(np.float32)
    return f32_to_bf16_bits(acc)


# --------------------------------------------------------------------------- #
# full FFN chain                                     gen_data_moe.py:552-707
# --------------------------------------------------------------------------- #
def moe_ffn(x_bits, expert_idx, probs, w1_codes, w1_scales, w2_codes, w2_scales, stages: bool = False):
    """dispatch -> quant -> GMM1 -> SwiGLU -> requant -> GMM2 -> combine on one
    device (EP = 1: both all-to-all steps are identities).

    x bf16 bits [T, K]; expert_idx int32 [T, topK]; probs fp32 [T, topK];
    w1 [E, N, K] + scales [E, N, K/32]; w2 [E, K, N/2] + scales [E, K, N/64].
    Returns bf16 bits [T, K] (and a dict of intermediates when ``stages``)."""
    x_bits = np.asarray(x_bits, dtype=np.uint16)
    t, k = x_bits.shape
    top_k = expert_idx.shape[1]
    e = w1_codes.shape[0]
    sorted2src, src2sorted, counts = moe_init_routing(expert_idx, e)
    xq, xs = mx_quant_bf16(x_bits, "E4M3", "rne")               # :574-585 (quantize once per token)
    src_tok = sorted2src.astype(np.int64) // top_k
    aq, asc = xq[src_tok], xs[src_tok]                            # :52-56 + alltoallv1 (EP=1)
    h, act, qa, sa = gmm1_swiglu_quant(aq, asc, w1_codes, w1_scales, counts)   # :646-658
    y = f32_to_bf16_bits(mx_gmm_f32(qa, sa, w2_codes, w2_scales, counts))      # :676-680
    out = unpermute_combine(y, src2sorted, probs)                 # device fp32 combine
    if stages:
        return out, dict(sorted2src=sorted2src, src2sorted=src2sorted, counts=counts, aq=aq, asc=asc,
                         h=h, act=act, qa=qa, sa=sa, y=y)
    return out


def unpermute_cpu_bf16(y_bits, sorted2src, probs) -> np.ndarray:
    """The golden's CPU fallback combine (gen_data_moe.py:60-70): bf16 multiply,
    bf16 ``index_add_`` in sorted-row order.  This is what the reference-made FFN vector
    (tests/golden/ffn_tiny.npz) was combined with; the product follows the device's fp32
    combine (:func:`unpermute_combine`) and stays inside the acceptance tolerance of this variant."""
    y = bf16_bits_to_f32(y_bits)
    probs = np.asarray(probs, dtype=np.float32)
    t, top_k = probs.shape
    out = np.zeros((t, y.shape[1]), dtype=np.float32)
    idx = np.asarray(sorted2src, dtype=np.int64)
    for i in range(idx.size):
        tok, kk = idx[i] // top_k, idx[i] % top_k
        w = bf16_round(np.float32(probs[tok, kk]))
        out[tok] = bf16_round(out[tok] + bf16_round(y[i] * w))
    return f32_to_bf16_bits(out)


# --------------------------------------------------------------------------- #
# acceptance rule                       verify_result.py:188-241, utils.py:97-105
# --------------------------------------------------------------------------- #
def get_rtol_bf16(compute_times: int) -> float:
    return 2.0 ** -7 if compute_times < 2048 else 2.0 ** -6


def verify_bf16(out_bits, golden_f32, k: int):
    """Reference acceptance for a bf16 output: every element within
    rtol*max(1,|golden|) and |mean(diff/max(1,|golden|))| <= 2^-7; non-finite
    positions must coincide.  Returns (ok, error_num, eb)."""
    out = bf16_bits_to_f32(out_bits).astype(np.float32).ravel()
    gold = np.asarray(golden_f32, dtype=np.float32).ravel()
    if np.count_nonzero(np.isfinite(out) != np.isfinite(gold)):
        return False, -1, float("inf")
    out = np.where(np.isfinite(out), out, 0)
    gold = np.where(np.isfinite(gold), gold, 0)
    rtol = get_rtol_bf16(k)
    diff = out - gold
    tmax = np.maximum(1.0, np.abs(gold))
    err = int(np.count_nonzero(np.abs(diff) - rtol * tmax > 0))
    eb = float(abs(np.mean(diff / tmax)))
    return (err == 0 and eb <= 2.0 ** -7), err, eb


def verify_double_golden_bf16(out_bits, golden_f32, golden_low_bits):
    """The double-golden acceptance of the dense MXFP8 matmul (verify_result.py:117-134, 244-306 with
    OpTypes.COMPUTE_FLOAT_HIGH_PRECISION and a bf16 output, as
    ascend950_mxfp8_matmul_reduce_scatter/scripts/run.sh:57-62 calls it): the output's maximum and mean relative
    error and its RMSE against the fp32 golden, each divided by max(the same figure of the bf16 "low" golden,
    2^-8), must stay below 10, 2 and 2, and |mean((out - gold) / max(1, |gold|))| <= 2^-7; non-finite positions
    must coincide.  Returns (ok, max_ratio, mean_ratio, rmse_ratio, eb)."""
    out = bf16_bits_to_f32(out_bits).astype(np.float32).ravel()
    gold = np.asarray(golden_f32, dtype=np.float32).ravel()
    low = bf16_bits_to_f32(golden_low_bits).astype(np.float32).ravel()
    if np.count_nonzero(np.isfinite(out) != np.isfinite(gold)):
        return False, float("inf"), float("inf"), float("inf"), 0.0
    out = np.where(np.isfinite(out), out, np.float32(0))
    gold = np.where(np.isfinite(gold), gold, np.float32(0))
    low = np.where(np.isfinite(low), low, np.float32(0))
    thr = np.float32(2.0 ** -8)
    eps = np.float32(1e-7)
    d_out, d_low = out - gold, low - gold
    eb = float(abs(np.mean(d_out / np.maximum(np.float32(1), np.abs(gold)))))
    rel_out, rel_low = np.abs(d_out) / (np.abs(gold) + eps), np.abs(d_low) / (np.abs(gold) + eps)
    rmse_out, rmse_low = np.sqrt(np.mean(d_out ** 2)), np.sqrt(np.mean(d_low ** 2))
    r_max = float(rel_out.max() / max(rel_low.max(), thr))
    r_mean = float(rel_out.mean() / max(rel_low.mean(), thr))
    r_rmse = float(rmse_out / max(rmse_low, thr))
    return (r_max < 10 and r_mean < 2 and r_rmse < 2 and eb <= 2.0 ** -7), r_max, r_mean, r_rmse, eb


# --------------------------------------------------------------------------- #
# host-side sizing contracts
# --------------------------------------------------------------------------- #
def _align(x: int, a: int) -> int:
    return (x + a - 1) // a * a


def moe_ready_swiglu_region_bytes(staging: int, local_experts: int) -> int:
    """include/catccos/detail/ascend950_moe_ready.hpp:44-49"""
    return _align(max(staging, local_experts * 64), 512)


def moe_ready_dispatch_region_bytes(staging: int, ranks: int, local_experts: int) -> int:
    """ascend950_moe_ready.hpp:38-42,51-56"""
    ready = _align(ranks * local_experts * 4, 64) + local_experts * 64
    return _align(max(staging, ready), 512)


def moe_ub_input_quant_bytes(hidden: int) -> int:
    """include/catccos/detail/ascend950_moe_ub.h:29-35"""
    scale = _align((hidden + 31) // 32, 2)
    return 2 * (3 * hidden + 5 * scale)


def moe_ub_dispatch_bytes(hidden: int) -> int:
    """ascend950_moe_ub.h:37-43"""
    scale = _align((hidden + 31) // 32, 2)
    row = _align(hidden + scale, 32)
    return 2 * _align(2 * row, 64)


def moe_ub_unpermute_bytes(m: int, hidden: int, top_k: int, aiv: int) -> int:
    """ascend950_moe_ub.h:45-55"""
    if aiv == 0:
        return 256 * 1024 + 1
    rows = max(1, min(m // aiv, 600))
    return 18 * _align(hidden, 512) + 256 + 2 * _align(rows * top_k * 4, 32)


def moe_ub_fits(m: int, hidden: int, top_k: int, aiv: int) -> bool:
    """ascend950_moe_ub.h:57-61"""
    cap = 256 * 1024
    return (moe_ub_input_quant_bytes(hidden) <= cap and moe_ub_dispatch_bytes(hidden) <= cap
            and moe_ub_unpermute_bytes(m, hidden, top_k, aiv) <= cap)


def ffn_workspace_bytes(m: int, k: int, n: int, rank_size: int, ep_size: int, expert_num: int, top_k: int) -> int:
    """Ascend950DispatchFFNCombineOperator::GetWorkspaceSize
    (ascend950_dispatch_ffn_combine_host.h:145-164)."""
    epr = expert_num // ep_size
    ep = rank_size
    rows = m * rank_size * top_k
    meta = ep * ep * epr * 4
    return (_align(_align(m, 256) * top_k * 4, 512) + _align(rows * k * 2, 512) + _align(meta, 512)
            + _align(rows * k, 512) + _align(rows * _align((k + 31) // 32, 2), 512)
            + moe_ready_swiglu_region_bytes(rows * (n // 2) * 2, epr)
            + _align(rows * (n // 2), 512) + _align(rows * _align((n // 2 + 31) // 32, 2), 512)
            + moe_ready_dispatch_region_bytes(rows * k * 2, ep, epr) + _align(meta, 512))


def balanced_expert_idx(m: int, expert_num: int, top_k: int, ep: int):
    """Round-robin routing generator (examples/utils/moe_routing.py:5-25)."""
    for name, v in (("m", m), ("expert_num", expert_num), ("top_k", top_k), ("ep", ep)):
        if v <= 0:
            raise ValueError(f"{name} must be positive, got {v}")
    if top_k > expert_num:
        raise ValueError(f"top_k ({top_k}) must not exceed expert_num ({expert_num})")
    base = np.arange(ep * m * top_k, dtype=np.int64).reshape(ep, m, top_k)
    return (base % expert_num).astype(np.int32)
