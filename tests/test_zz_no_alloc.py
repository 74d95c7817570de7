"""The allocation-free entry point cmx_mx_gmm_swiglu_quant_noalloc against cmx_mx_gmm_swiglu_quant: same codes, scales
and bf16 activations bit for bit, on two calls in a row (the second with a smaller input, so that it runs on what
the first left in the library's static schedule array), with no device allocation in between."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O
from tests.gpu_util import dev, host

pytestmark = pytest.mark.gpu


def _case(seed, counts, n, k):
    rng = np.random.default_rng(seed)
    m = sum(counts)
    aq, asc = O.mx_quant(O.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))
    qs = [O.mx_quant(O.bf16_round(rng.standard_normal((n, k)).astype(np.float32) * 0.06), "E4M3", "lut") for _ in counts]
    return dev(aq), dev(asc), dev(np.stack([q for q, _ in qs])), dev(np.stack([s for _, s in qs])), dev(np.array(counts, dtype=np.int32))


def test_noalloc_entry_point_matches_the_workspace_one_on_two_calls_in_a_row():
    from catccos_amd import ops
    ops.init()
    big = _case(1, [300, 0, 257, 5, 700, 0, 64, 1, 130], 512, 1024)
    small = _case(2, [0, 40, 3], 256, 512)
    # everything torch allocates (expected results, output buffers) exists before the first free-memory reading; a first
    # call on a case of its own has loaded whatever the runtime loads lazily
    warm = _case(3, [33], 128, 512)
    ops.mx_gmm_swiglu_quant_noalloc(*warm[:4], warm[4], 512, torch.empty((33, 64), dtype=torch.uint8, device="cuda"),
                                    torch.empty((33, 2), dtype=torch.uint8, device="cuda"), torch.empty((33, 64), dtype=torch.bfloat16, device="cuda"))
    ops.mx_gmm_swiglu_quant_noalloc(*warm[:4], warm[4], 512, torch.empty((33, 64), dtype=torch.uint8, device="cuda"),
                                    torch.empty((33, 2), dtype=torch.uint8, device="cuda"), None)
    prepared = []
    for a, a_s, w, w_s, cnt in (big, small):
        m, n, k = a.shape[0], w.shape[1], a.shape[1]
        want = ops.mx_gmm_swiglu_quant(a, a_s, w, w_s, cnt, k, want_bf16=True)
        codes = torch.full((m, n // 2), 0xEE, dtype=torch.uint8, device="cuda")
        scales = torch.full((m, ops.scale_cols(n // 2)), 0xEE, dtype=torch.uint8, device="cuda")
        act = torch.full((m, n // 2), 7.0, dtype=torch.bfloat16, device="cuda")
        codes2, scales2 = codes.clone(), scales.clone()
        prepared.append((a, a_s, w, w_s, cnt, k, want, codes, scales, act, codes2, scales2))
    torch.cuda.synchronize()
    # free device memory as the driver reports it: a hipMalloc, hipMallocAsync or hipFree inside the library would move
    # it (torch's own counters only see torch's allocator)
    free_before = torch.cuda.mem_get_info()[0]
    torch_before = torch.cuda.memory_allocated()
    for a, a_s, w, w_s, cnt, k, want, codes, scales, act, codes2, scales2 in prepared:
        ops.mx_gmm_swiglu_quant_noalloc(a, a_s, w, w_s, cnt, k, codes, scales, act)        # with the bf16 output
        ops.mx_gmm_swiglu_quant_noalloc(a, a_s, w, w_s, cnt, k, codes2, scales2, None)     # the benchmarked instantiation
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == torch_before
    for a, a_s, w, w_s, cnt, k, (want_codes, want_scales, want_act), codes, scales, act, codes2, scales2 in prepared:
        assert torch.equal(codes, want_codes) and torch.equal(scales, want_scales)
        assert torch.equal(act.view(torch.int16), want_act.view(torch.int16))
        assert torch.equal(codes2, want_codes) and torch.equal(scales2, want_scales)
        # and against the oracle: the codes are what the oracle quantizer makes of the kernel's bf16 output
        q2, s2 = O.mx_quant_bf16(host(want_act), "E4M3", "rne")
        assert np.array_equal(host(codes2), q2) and np.array_equal(host(scales2), s2)


def test_noalloc_entry_point_rejects_more_groups_than_its_array_holds():
    from catccos_amd import _lib
    lib = _lib.load()
    limit = lib.cmx_mx_gmm_noalloc_max_groups()
    assert limit == 4096
    z = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    rc = lib.cmx_mx_gmm_swiglu_quant_noalloc(p, 256, p, 8, p, p, p, 64, p, 2, None, p, limit + 1, 16, 128, 256, None)
    assert rc == -1 and b"4096" in lib.cmx_last_error()
