"""Helpers shared by the GPU parity tests (tests marked `gpu` call libmk_hip.so through its C ABI)."""
import numpy as np


def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    return torch


def dev(a):
    torch = torch_cuda()
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_l2(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-300))
