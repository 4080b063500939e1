"""Helpers shared by the GPU parity tests."""
import sys

import numpy as np
import torch


def announce(*what):
    """Name the case before the GPU step, flushed: if the step takes the box down this line survives."""
    print('[gpu-case]', *what, flush=True)
    sys.stdout.flush()


def dev(x: np.ndarray, dtype=None) -> torch.Tensor:
    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def host(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.float().cpu().numpy()
    return t.cpu().numpy()
