"""Helpers shared by the GPU parity tests (not collected by pytest)."""
import numpy as np
import torch


def dev():
    return torch.device("cuda:0")


def to_dev_bits(a):
    """uint16 bf16 bits -> int16 device tensor."""
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(dev())


def rel_err(got, ref):
    """max |got - ref| scaled by the largest reference magnitude (outputs of one matvec share a scale)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))
