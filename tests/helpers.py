"""Shared test plumbing: numpy <-> device tensors for BF16/FP8 bit patterns, error measures."""

import ctypes as ct

import numpy as np
import torch

import oracle


def to_device_bf16(bits, device):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).to(device)


def from_device_bf16(tensor):
    return tensor.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def to_device_fp8(bytes_, device):
    return torch.from_numpy(np.ascontiguousarray(bytes_)).view(torch.float8_e4m3fn).to(device)


def from_device_fp8(tensor):
    return tensor.detach().cpu().contiguous().view(torch.uint8).numpy()


def bf16_values(tensor):
    return oracle.bf16_to_f32(from_device_bf16(tensor))


def rel_frobenius(got, want):
    return oracle.rel_frobenius(got, want)


def bf16_ulp_distance(a_bits, b_bits):
    """Distance in BF16 units-in-the-last-place between two bit-pattern arrays (finite values)."""

    def ordered(bits):
        bits = bits.astype(np.int32)
        return np.where(bits & 0x8000, 0x8000 - (bits & 0x7FFF) - 1, bits + 0x8000 - 0)

    return np.abs(ordered(a_bits) - ordered(b_bits))


def ptr(tensor):
    return ct.c_void_p(tensor.data_ptr()) if tensor is not None else None
