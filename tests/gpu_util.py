"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(x):
    """numpy -> device tensor keeping the bits (uint16 half/bf16 need a dtype)."""
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def half_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.float16)).cuda()


def bf16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)


def half_bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def ulp_distance_16(a_bits, b_bits):
    """Distance in representable values between two arrays of half or bf16 bits."""
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7fff), b & 0x7fff)
    return np.abs(key(a_bits) - key(b_bits))
