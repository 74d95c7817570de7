"""ctypes binding of libcatccos_mx.so (the C ABI declared in include/catccos_mx.h).

The library is loaded from catccos_amd/lib/; nothing here falls back to another
implementation: a missing library raises ImportError with the build command.
"""
from __future__ import annotations

import ctypes as C
import os

import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_LIB_PATH = os.path.join(_HERE, "lib", "libcatccos_mx.so")
# CATCCOS_MX_LIB points at another build of the same library (e.g. an experimental kernel variant); load() says so
# on stderr, so that no run uses a substitute unnoticed
LIB_PATH = os.environ.get("CATCCOS_MX_LIB") or DEFAULT_LIB_PATH

u8p, i32p, f32p, vp = C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p
u32, i32, u64, sz = C.c_uint32, C.c_int, C.c_uint64, C.c_size_t


class FfnWorkspaceLayout(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in (
        "src2sorted", "sorted2src", "counts", "routing_scratch", "gmm_meta",
        "a_codes", "a_scales", "act_codes", "act_scales", "y", "total", "a_scales_pitch")]


# name -> (restype, argtypes); every symbol include/catccos_mx.h declares
SIGNATURES = {
    "cmx_version": (i32, []),
    "cmx_last_error": (C.c_char_p, []),
    "cmx_rt_device_count": (i32, [C.POINTER(C.c_int)]),
    "cmx_rt_set_device": (i32, [i32]),
    "cmx_rt_malloc": (i32, [C.POINTER(C.c_void_p), sz]),
    "cmx_rt_free": (i32, [vp]),
    "cmx_rt_malloc_host": (i32, [C.POINTER(C.c_void_p), sz]),
    "cmx_rt_free_host": (i32, [vp]),
    "cmx_rt_memcpy_h2d": (i32, [vp, vp, sz]),
    "cmx_rt_memcpy_d2h": (i32, [vp, vp, sz]),
    "cmx_rt_memset": (i32, [vp, i32, sz]),
    "cmx_rt_stream_create": (i32, [C.POINTER(C.c_void_p)]),
    "cmx_rt_stream_destroy": (i32, [vp]),
    "cmx_rt_stream_sync": (i32, [vp]),
    "cmx_mx_quant": (i32, [vp, u32, u8p, u32, u8p, u32, u32, u32, i32, i32, vp]),
    "cmx_mx_dequant": (i32, [u8p, u32, u8p, u32, f32p, u32, u32, u32, i32, vp]),
    "cmx_mx_gemm": (i32, [u8p, u32, u8p, u32, u8p, u32, u8p, u32, vp, u32, u32, u32, u32, i32, i32, vp]),
    "cmx_mx_gmm_workspace_bytes": (sz, [u32]),
    "cmx_mx_gmm": (i32, [u8p, u32, u8p, u32, u8p, u8p, vp, u32, i32p, u32, u32, u32, u32, i32, i32, vp, vp]),
    "cmx_mx_gmm_swiglu_quant": (i32, [u8p, u32, u8p, u32, u8p, u8p, u8p, u32, u8p, u32, vp, i32p, u32, u32, u32, u32,
                                      vp, vp]),
    "cmx_mx_to_k_major": (i32, [u8p, u32, u8p, u8p, u32, u8p, u32, u32, u32, u32, vp]),
    "cmx_mxfp4_to_k_major": (i32, [u8p, u32, u8p, u8p, u32, u8p, u32, u32, u32, u32, vp]),
    "cmx_mx_gemm_ex_workspace_bytes": (sz, [u32, u32, u32, i32, i32]),
    "cmx_mx_gemm_ex": (i32, [u8p, u8p, u8p, u8p, vp, u32, u32, u32, u32, i32, i32, i32, i32, vp, vp]),
    "cmx_mx_gmm_ex_workspace_bytes": (sz, [u32, u32, u32, i32]),
    "cmx_mx_gmm_ex": (i32, [u8p, u8p, u8p, u8p, vp, u32, i32p, u32, u32, u32, u32, i32, i32, i32, vp, vp]),
    "cmx_int8_quant_scatter": (i32, [vp, u32, i32p, vp, u32, f32p, u32, u32, u32, vp]),
    "cmx_bytes_to_k_major": (i32, [u8p, u32, u8p, u32, u32, u32, u32, vp]),
    "cmx_int8_gmm_workspace_bytes": (sz, [u32, u32, u32, i32]),
    "cmx_int8_gmm_dequant_swiglu": (i32, [vp, u32, f32p, vp, f32p, u32, vp, u32, i32, i32p, u32, u32, u32, u32, i32, vp, vp]),
    "cmx_moe_routing_workspace_bytes": (sz, [u32, u32]),
    "cmx_moe_init_routing": (i32, [i32p, u32, u32, u32, i32p, i32p, i32p, vp, vp]),
    "cmx_packed_row_bytes": (u32, [u32]),
    "cmx_quant_scatter": (i32, [vp, u32, i32p, u8p, u32, u8p, u32, u32, u32, u32, vp]),
    "cmx_moe_token_unpermute": (i32, [vp, u32, u32, i32p, f32p, vp, u32, u32, u32, u32, vp]),
    "catccos_ascend950_symmetric_bytes": (u64, []),
    "catccos_ascend950_dispatch_ffn_combine_workspace_bytes": (sz, [u32, u32, u32, u32, u32, i32]),
    "catccos_ascend950_dispatch_ffn_combine": (i32, [u32, vp, u64, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u8p,
                                                     u32, u32, u32, u32, u32, i32]),
    "cmx_ffn_workspace_layout_get": (i32, [u32, u32, u32, u32, u32, C.POINTER(FfnWorkspaceLayout)]),
    "cmx_mx_pretiled_weight_bytes": (sz, [u32, u32, u32, i32]),
    "cmx_mx_pretile_weights": (i32, [u8p, u8p, u32, u32, u32, i32, vp]),
    "cmx_mx_gmm_pretiled": (i32, [u8p, u32, u8p, u32, u8p, u8p, vp, u32, i32p, u32, u32, u32, u32, i32, i32, vp, vp]),
    "cmx_mx_gmm_swiglu_quant_pretiled": (i32, [u8p, u32, u8p, u32, u8p, u8p, u8p, u32, u8p, u32, vp, i32p, u32, u32,
                                               u32, u32, vp, vp]),
    "cmx_dispatch_ffn_combine_pretiled": (i32, [vp, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u8p, u32, u32, u32, u32,
                                                u32]),
    "cmx_init": (i32, []),
    "cmx_mx_gmm_noalloc_max_groups": (u32, []),
    "cmx_mx_gmm_swiglu_quant_noalloc": (i32, [u8p, u32, u8p, u32, u8p, u8p, u8p, u32, u8p, u32, vp, i32p, u32, u32, u32,
                                              u32, vp]),
}

_lib = None


def bind(path: str, extra_signatures=None) -> C.CDLL:
    """Loads the shared library at ``path`` and types every entry point of the C ABI (plus ``extra_signatures``)."""
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m catccos_amd.build` (needs hipcc). "
            "There is no CPU fallback.")
    lib = C.CDLL(path)
    for name, (res, args) in {**SIGNATURES, **(extra_signatures or {})}.items():
        fn = getattr(lib, name)          # AttributeError names the missing symbol
        fn.restype = res
        fn.argtypes = args
    return lib


def load() -> C.CDLL:
    """The library every function of the package calls."""
    global _lib
    if _lib is None:
        if LIB_PATH != DEFAULT_LIB_PATH:
            print(f"catccos_amd: CATCCOS_MX_LIB overrides the library: loading {LIB_PATH}", file=sys.stderr)
        _lib = bind(LIB_PATH)
    return _lib


def activate(lib) -> "C.CDLL | None":
    """Makes ``lib`` (a result of bind(), or None for the default) the library that load() returns; returns the
    previous one.  The test suite uses it to run the package's front end on the test build of the library."""
    global _lib
    prev, _lib = _lib, lib
    return prev


class CmxError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc != 0:
        msg = load().cmx_last_error()
        raise CmxError(f"libcatccos_mx error {rc}: {msg.decode() if msg else ''}")
