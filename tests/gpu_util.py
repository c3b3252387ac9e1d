"""Shared helpers of the GPU parity tests: numpy <-> device tensors with the reference's dtypes."""
import numpy as np
import torch

DEV = "cuda:0"


def t_f16(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float16)).to(DEV)


def t_u32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint32).view(np.int32)).to(DEV).view(torch.uint32)


def t_u16(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint16).view(np.int16)).to(DEV).view(torch.uint16)


def t_bf16_bits(bits):
    return t_u16(bits).view(torch.bfloat16)


def n_u32(t):
    return t.cpu().view(torch.int32).numpy().view(np.uint32)


def n_u16(t):
    return t.cpu().view(torch.int16).numpy().view(np.uint16)


def n_f16(t):
    return t.cpu().numpy()


def n_bf16_bits(t):
    return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def bf16_bits(x_f32):
    """fp32 numpy -> bf16 bit patterns (round to nearest even) via torch on the CPU"""
    return torch.from_numpy(np.ascontiguousarray(x_f32, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
