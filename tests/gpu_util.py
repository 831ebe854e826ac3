"""Helpers for the GPU parity tests (torch is only the device allocator)."""
import numpy as np
import torch


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda")


def host(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy()


def say(*a):
    # name the case before its kernels run, so a fault can be attributed
    print("[case]", *a, flush=True)
