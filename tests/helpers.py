"""Shared helpers for the parity tests: seeded inputs and bit-level views."""
import numpy as np


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def bits16(t):
    """uint16 bit patterns of a torch f16/bf16 tensor, as a flat numpy array."""
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16).ravel()


def from_bits16(bits, torch_dtype, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch_dtype).to(device)


def f32_bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).ravel()


def torch_dtype_of(orc, dtype):
    import torch
    return {orc.F32: torch.float32, orc.F16: torch.float16, orc.BF16: torch.bfloat16}[dtype]


def to_device_float(orc, x_f32, dtype, device):
    """Host f32 values -> (device tensor of `dtype`, numpy storage array as the oracle reads it)."""
    import torch
    if dtype == orc.F32:
        a = np.ascontiguousarray(x_f32, dtype=np.float32)
        return torch.from_numpy(a).to(device), a.ravel()
    bits = orc.narrow(x_f32, dtype)
    return from_bits16(bits, torch_dtype_of(orc, dtype), device).reshape(x_f32.shape), bits.ravel()


def float_storage(orc, t, dtype):
    """Device float tensor -> numpy storage array in the oracle's representation."""
    if dtype == orc.F32:
        return t.cpu().numpy().ravel()
    return bits16(t)
