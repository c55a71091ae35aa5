"""Helpers shared by the GPU parity tests: numpy <-> device tensors, error norms."""
import numpy as np
import torch

DEV = "cuda:0"


def dev(a):
    """numpy array -> device tensor (uint16 arrays of bf16 / fp16 bits stay integer-typed via int16 views)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def dev_bf16(bits):
    return dev(bits).view(torch.bfloat16)


def dev_f16(bits):
    return dev(bits).view(torch.float16)


def host(t):
    t = t.detach().cpu()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def rel_l2(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
