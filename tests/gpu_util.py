"""Helpers for the GPU parity tests."""
import numpy as np
import torch


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    return t.detach().float().cpu().numpy()


def bf16_round(a):
    """float32 array rounded to the nearest bf16 value (returned as float32)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).float().numpy()


def round_to(a, dtype):
    """float32 array rounded to the nearest value of a torch storage type (returned as float32)."""
    if dtype == torch.float32:
        return np.ascontiguousarray(a, dtype=np.float32)
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).float().numpy()
