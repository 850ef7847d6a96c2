"""Helpers shared by the GPU parity tests: numpy <-> device buffers and the tolerance."""
import numpy as np
import torch

# max over elements of |d - ref| / max(|ref|, 1e-2 * rms(ref)); the bar for every GEMM output
GEMM_TOL = 1e-2


def dev(a):
    """numpy array -> CUDA tensor with the matching torch dtype (uint16 is carried as bf16 bits)."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bits(t):
    """bf16 CUDA tensor -> numpy uint16 bit patterns."""
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16)


def scale_tensor(s):
    return torch.tensor([float(s)], dtype=torch.float32, device="cuda")
