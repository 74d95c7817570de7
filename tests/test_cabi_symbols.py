"""The C-ABI library loads without a GPU and exports exactly what include/catccos_mx.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "catccos_mx.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # drop comments
    text = re.sub(r"//[^\n]*", "", text)
    names = re.findall(r"\b((?:cmx|catccos_ascend950)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("cmx_mx_quant", "cmx_mx_dequant", "cmx_mx_gemm", "cmx_mx_gmm", "cmx_mx_gmm_swiglu_quant", "cmx_moe_init_routing",
                 "cmx_quant_scatter", "cmx_moe_token_unpermute", "catccos_ascend950_dispatch_ffn_combine",
                 "catccos_ascend950_dispatch_ffn_combine_workspace_bytes", "catccos_ascend950_symmetric_bytes"):
        assert must in names
    assert len(names) >= 25


def test_library_exports_every_declared_symbol():
    from catccos_amd import _lib
    lib = _lib.load()
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, missing
    # the ctypes table of the Python front end covers the same set
    assert sorted(_lib.SIGNATURES) == _declared()


def test_host_only_entry_points_work_without_a_gpu():
    from catccos_amd import _lib
    lib = _lib.load()
    assert lib.cmx_version() >= 1
    assert lib.catccos_ascend950_symmetric_bytes() == 1004 * 1024 * 1024
    assert lib.cmx_packed_row_bytes(7168) == 7168 + 224
    # a bad argument is reported through the error string, not a crash
    rc = lib.cmx_mx_quant(None, 0, None, 0, None, 0, 1, 33, 0, 0, None)
    assert rc != 0 and lib.cmx_last_error()
    # the pre-tiled family validates on the host before anything is launched
    assert lib.cmx_mx_pretile_weights(None, None, 2, 256, 512, 0, None) == -1 and b"null pointer" in lib.cmx_last_error()
    assert lib.cmx_mx_pretile_weights(16, 32, 2, 256, 256, 0, None) == -1 and b"multiple of 512" in lib.cmx_last_error()
    assert lib.cmx_mx_pretile_weights(16, 32, 2, 96, 512, 1, None) == -1 and b"multiple of 64" in lib.cmx_last_error()
    assert lib.cmx_mx_pretile_weights(8, 32, 2, 256, 512, 0, None) == -1 and b"16-byte aligned" in lib.cmx_last_error()
    assert lib.cmx_mx_pretile_weights(None, None, 0, 256, 512, 0, None) == 0           # nothing to do
    assert lib.cmx_dispatch_ffn_combine_pretiled(None, 16, 16, 16, 16, 16, 16, 16, 16, 256, 8, 512, 512, 4, 2) == -1
    assert b"N % 1024" in lib.cmx_last_error()
    assert lib.cmx_dispatch_ffn_combine_pretiled(None, 16, 16, 16, 16, 16, 16, 16, 16, 256, 8, 768, 1024, 4, 2) == -1


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 (and as C++) on its own."""
    import subprocess
    for compiler, std, lang in (("gcc", "-std=c99", "c"), ("g++", "-std=c++17", "c++")):
        r = subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", lang, HEADER],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr


def test_workspace_sizes_are_host_arithmetic():
    from catccos_amd import _lib
    lib = _lib.load()
    assert lib.cmx_mx_gemm_ex_workspace_bytes(100, 200, 512, 0, 1) == 0                    # both operands K-contiguous
    need = lib.cmx_mx_gemm_ex_workspace_bytes(100, 200, 512, 1, 0)
    assert need >= (100 + 200) * (512 + 16) and need % 256 == 0
    meta = lib.cmx_mx_gmm_workspace_bytes(16)
    assert lib.cmx_mx_gmm_ex_workspace_bytes(16, 256, 512, 1) >= meta
    assert lib.cmx_mx_gmm_ex_workspace_bytes(16, 256, 512, 0) >= meta + 16 * 256 * (512 + 16)
    assert lib.cmx_int8_gmm_workspace_bytes(4, 256, 512, 0) >= lib.cmx_int8_gmm_workspace_bytes(4, 256, 512, 1) + 4 * 256 * 512
    # pre-tiled weights: whole 256-row tiles (gate|up weights: 128 + 128 rows), 0 for shapes the layout does not cover
    assert lib.cmx_mx_pretiled_weight_bytes(256, 4096, 7168, 1) == 256 * 4096 * 7168
    assert lib.cmx_mx_pretiled_weight_bytes(3, 320, 512, 0) == 3 * 512 * 512
    assert lib.cmx_mx_pretiled_weight_bytes(2, 640, 1024, 1) == 2 * 3 * 256 * 1024
    assert lib.cmx_mx_pretiled_weight_bytes(2, 640, 256, 0) == 0 and lib.cmx_mx_pretiled_weight_bytes(2, 96, 512, 1) == 0
