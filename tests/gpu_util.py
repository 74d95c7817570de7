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
