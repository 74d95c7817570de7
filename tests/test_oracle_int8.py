"""Pins the INT8 W8A8 oracle (oracle/int8_oracle.py) against integer brute force and torch CPU library ops."""
import numpy as np
import torch

from oracle import int8_oracle as Q


def test_dynamic_quant_known_answers_and_torch_formula():
    x = np.array([[1.0, -2.0, 0.5, 0.0], [0.0, 0.0, 0.0, 0.0], [3.0, 1.5, -3.0, 0.0118110236]], dtype=np.float32)
    q, s = Q.dynamic_quant(x)
    assert q[0].tolist() == [64, -127, 32, 0]            # 63.5 -> 64 and 31.75 -> 32 (half to even / nearest)
    assert q[1].tolist() == [0, 0, 0, 0] and s[1] == 0
    assert q[2].tolist() == [127, 64, -127, 0]           # 63.5 -> 64 (even), 0.4999.. -> 0
    assert s[0] == np.float32(2.0) / np.float32(127.0)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((64, 96)).astype(np.float32)
    t = torch.from_numpy(x)
    mx = torch.max(torch.abs(t), dim=-1).values
    want = torch.round(t * 127. / mx[:, None]).to(torch.int8).numpy()      # the generator's helper, verbatim ops
    q, s = Q.dynamic_quant(x)
    assert np.array_equal(q, want) and np.array_equal(s, (mx / 127.).numpy())
    assert np.abs(q).max() == 127 and np.all(np.abs(q.astype(np.int32)).max(axis=1) == 127)


def test_int32_matmul_is_exact_against_python_integers():
    rng = np.random.default_rng(1)
    a = rng.integers(-128, 128, size=(3, 64), dtype=np.int8)
    b = rng.integers(-128, 128, size=(1, 64, 4), dtype=np.int8)
    ones = np.ones(3, dtype=np.float32)
    # unit scales, columns [x0 | gate]: recover c through gate when x0 is huge (sigmoid -> 1): use the dequant directly
    c = a.astype(np.int32) @ b[0].astype(np.int32)
    for i in range(3):
        for j in range(4):
            assert int(c[i, j]) == sum(int(a[i, t]) * int(b[0, t, j]) for t in range(64))
    # extremes stay inside int32 at the largest K of the path
    k = 7168
    assert 128 * 128 * k < 2 ** 31
    out = Q.gmm_dequant_swiglu(a, ones, b, np.full(4, 2.0 ** -10, dtype=np.float32), [3])
    h = (c.astype(np.float32) * np.float32(2.0 ** -10)).astype(np.float16).astype(np.float32)
    want = h[:, :2] / (1 + np.exp(-h[:, :2])) * h[:, 2:]
    assert np.allclose(out, want, rtol=1e-6, atol=1e-7)


def test_chain_against_torch_library_ops():
    rng = np.random.default_rng(2)
    counts = [5, 0, 9, 2]
    e, k, n = 4, 128, 64
    rows = sum(counts)
    a = rng.integers(-16, 16, size=(rows, k), dtype=np.int8)
    b = rng.integers(-16, 16, size=(e, k, n), dtype=np.int8)
    ch = Q.truncate_scale(rng.standard_normal(e * n).astype(np.float32) / 127)
    ts = (np.abs(rng.standard_normal(rows)) / 127).astype(np.float32)
    got = Q.gmm_dequant_swiglu(a, ts, b, ch, counts)
    outs, r0 = [], 0
    for g, cnt in enumerate(counts):
        c = torch.matmul(torch.from_numpy(a[r0:r0 + cnt]).to(torch.int32), torch.from_numpy(b[g]).to(torch.int32))
        h = (c.to(torch.float32) * torch.from_numpy(ch.reshape(e, n)[g])[None, :]).to(torch.float16)
        y = h.to(torch.float32) * torch.from_numpy(ts[r0:r0 + cnt])[:, None]
        x0, gate = y.chunk(2, dim=-1)
        outs.append(x0 * torch.sigmoid(x0) * gate)
        r0 += cnt
    want = torch.cat(outs).numpy()
    assert np.allclose(got, want, rtol=2e-6, atol=1e-9)
    # the fp16 step is a real rounding: leaving it out changes the result
    y32 = np.concatenate([(a[:5].astype(np.int32) @ b[0].astype(np.int32)).astype(np.float32) * ch.reshape(e, n)[0][None, :]])
    assert not np.array_equal(y32.astype(np.float16).astype(np.float32), y32)


def test_scale_file_words_and_truncation():
    ch = np.array([0.5, -1.25e-3, 3.0], dtype=np.float32)
    w = Q.channel_scale_words(ch)
    assert w.dtype == np.int64 and np.array_equal(w.view(np.float32)[0::2], ch) and np.all(w.view(np.int32)[1::2] == 0)
    t = Q.truncate_scale(np.array([1.0 + 2.0 ** -20, 0.3], dtype=np.float32))
    assert t[0] == 1.0 and (t.view(np.int32) & 0x1FFF).max() == 0


def test_dispatch_quant_follows_the_sort():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 32)).astype(np.float32)
    idx = rng.integers(0, 4, size=(6, 2))
    order = np.argsort(idx.reshape(-1), kind="stable")
    q, s = Q.dispatch_quant(x, order, 2)
    q0, s0 = Q.dynamic_quant(x)
    for i, src in enumerate(order):
        assert np.array_equal(q[i], q0[src // 2]) and s[i] == s0[src // 2]
