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


def bf16_safe(v64, margin=4e-6, size=None):
    """True where rounding v64 (binary64) to bf16 cannot be changed by an error below `margin` times the value's size (`size`; its
    own magnitude unless given, e.g. the norm of a sum's terms): the value is not that close to the midpoint of two neighbouring bf16
    values.  Lets a test demand equal bits from two binary32 evaluations of one expression whose library exponentials or orders
    of summation may differ in the last places."""
    t = torch.from_numpy(np.ascontiguousarray(v64, np.float64))
    lo = t.to(torch.float32).to(torch.bfloat16).double()
    _, ex = torch.frexp(torch.where(lo == 0, torch.full_like(lo, 2.0 ** -126), lo))      # |lo| in [2^(ex-1), 2^ex): a bf16 step there is 2^(ex-8)
    half = torch.pow(2.0, ex.double() - 9)
    half = torch.where((t.abs() < lo.abs()) & (lo.abs() == torch.pow(2.0, ex.double() - 1)), half / 2, half)   # below a power of two the steps are half as wide
    dist = ((t - lo).abs() - half).abs()                # distance to the rounding boundary on the side the value lies on
    sz = t.abs() if size is None else torch.from_numpy(np.ascontiguousarray(size, np.float64))
    return ((dist > margin * sz) | (sz == 0)).numpy()
