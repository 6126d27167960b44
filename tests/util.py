"""Shared helpers for the parity tests."""
import numpy as np
import torch


def key16(t):
    """fp16/bf16 tensor -> monotone integer per element (distance = units in the last place)."""
    i = t.view(torch.int16).int()
    return torch.where(i < 0, -(i & 0x7FFF), i)


def ulp16(a, b):
    return (key16(a) - key16(b)).abs()


def close16(got, want, max_ulp=1, atol=0.0):
    """Each element within max_ulp units in the last place of `want`, or within atol."""
    got, want = got.cpu(), want.cpu()
    ok = (ulp16(got, want) <= max_ulp) | ((got.float() - want.float()).abs() <= atol)
    return bool(ok.all())


def bf16_bits(t):
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bits_bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def to_np(t):
    """torch CPU tensor -> array the oracle takes (bf16 as uint16 bits), plus the dtype tag."""
    t = t.cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return bf16_bits(t), "bf16"
    return t.numpy(), None


def from_np(a, like_dtype):
    if like_dtype == torch.bfloat16:
        return bits_bf16(a)
    return torch.from_numpy(np.ascontiguousarray(a))


def rel_err(got, want):
    """max |got - want| / max |want| in double."""
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-300)).item()
