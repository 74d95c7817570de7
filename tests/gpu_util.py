"""Helpers shared by the GPU parity tests (numpy <-> device tensors)."""
import numpy as np
import torch


def dev(a: np.ndarray) -> torch.Tensor:
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def host(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.int16:
        return t.numpy().view(np.uint16)
    return t.numpy()


def bf16_dev(bits: np.ndarray) -> torch.Tensor:
    return dev(bits).view(torch.bfloat16)


def close_bf16(out_bits, gold_f32, rtol=1e-2, atol=1e-2):
    """|out - gold| <= atol + rtol*|gold| for every element (bf16 output vs fp32 golden)."""
    from oracle import mx_oracle as O
    out = O.bf16_bits_to_f32(out_bits).astype(np.float64)
    gold = np.asarray(gold_f32, dtype=np.float64)
    bad = np.abs(out - gold) > atol + rtol * np.abs(gold)
    return int(bad.sum()), float(np.abs(out - gold).max())


# ---- the test build of the library (tests/build_test_lib.py): the product's kernels plus the test hooks ----------
import ctypes as _C
import os as _os

TEST_LIB_PATH = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "lib", "libcatccos_mx_test.so")
_HOOKS = {
    "cmx_mfma_raw_probe": (_C.c_int, [_C.c_void_p] * 5 + [_C.c_int] * 3 + [_C.c_void_p]),
    "cmx_debug_force_tile": (_C.c_int, [_C.c_int] * 3),
    "cmx_debug_disable_streaming": (_C.c_int, [_C.c_int]),
    "cmx_debug_pretiled_tile_rows": (_C.c_int, [_C.c_int]),
}
_test_lib = None


def hooks_lib():
    """libcatccos_mx_test.so, typed like the product library plus the hooks."""
    global _test_lib
    if _test_lib is None:
        from catccos_amd import _lib
        if not _os.path.exists(TEST_LIB_PATH):
            raise ImportError(f"{TEST_LIB_PATH} is missing: build it with `python tests/build_test_lib.py`")
        _test_lib = _lib.bind(TEST_LIB_PATH, _HOOKS)
    return _test_lib


class hooked_library:
    """Context manager: the package's front end (catccos_amd.ops) runs on the test build while it is active."""

    def __enter__(self):
        from catccos_amd import _lib
        self.lib = hooks_lib()
        self.prev = _lib.activate(self.lib)
        return self.lib

    def __exit__(self, *exc):
        from catccos_amd import _lib
        self.lib.cmx_debug_force_tile(0, 0, 0)
        self.lib.cmx_debug_disable_streaming(0)
        self.lib.cmx_debug_pretiled_tile_rows(0)
        _lib.activate(self.prev)
        return False


def mfma_raw_probe(a_regs, b_regs, sa, sb, fmt: str, opsel: int, shape: int) -> torch.Tensor:
    from catccos_amd import _lib, ops
    out = torch.zeros((64, 16 if shape == 0 else 4), dtype=torch.float32, device=a_regs.device)
    rc = hooks_lib().cmx_mfma_raw_probe(a_regs.data_ptr(), b_regs.data_ptr(), sa.data_ptr(), sb.data_ptr(), out.data_ptr(),
                                       ops.FMT[fmt], opsel, shape, torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise _lib.CmxError(f"cmx_mfma_raw_probe failed: {hooks_lib().cmx_last_error().decode()}")
    return out
