"""Helpers of the GPU parity tests: seeded inputs generated on the CPU in fp32, rounded to
the activation dtype once, so that the HIP path and the fp64 oracle see identical bits."""
import numpy as np
import torch

DEV = "cuda:0"
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 4e-3}


def rounded(a: np.ndarray, dtype: torch.dtype):
    """(device tensor of `dtype`, the same values as float64 numpy)."""
    t = torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(dtype)
    return t.to(DEV), t.to(torch.float64).numpy()


def dev(a, dtype=torch.float32):
    a = np.asarray(a)
    if np.iscomplexobj(a):
        return torch.from_numpy(np.ascontiguousarray(a.astype(np.complex64))).to(DEV)
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(DEV)


def host(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.is_complex():
        return t.to(torch.complex128).numpy()
    if t.dtype in (torch.int64, torch.int32, torch.bool, torch.uint8):
        return t.numpy()
    return t.to(torch.float64).numpy()
