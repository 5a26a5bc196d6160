"""Helpers shared by the GPU parity tests: moving oracle bit patterns to the device."""
import numpy as np
import torch

_VIEW = {"f16": torch.float16, "bf16": torch.bfloat16}


def to_dev(bits, kind):
    """numpy bit patterns -> cuda tensor.  kind: 'f16' | 'bf16' | 'f8' | 'u32' | 'f32'."""
    bits = np.ascontiguousarray(bits)
    if kind in _VIEW:
        return torch.from_numpy(bits.view(np.int16)).view(_VIEW[kind]).cuda()
    if kind == "f8":
        return torch.from_numpy(bits).view(torch.float8_e4m3fn).cuda()
    if kind == "u32":
        return torch.from_numpy(bits.view(np.int32)).cuda()
    if kind == "f32":
        return torch.from_numpy(bits).cuda()
    raise ValueError(kind)


def to_bits(t):
    """cuda tensor -> numpy bit patterns (uint16 for 16-bit floats, uint8 for fp8)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    if t.dtype == torch.int32:
        return t.numpy().view(np.uint32)
    return t.numpy()
