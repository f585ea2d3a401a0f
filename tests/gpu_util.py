"""Helpers shared by the GPU parity tests: move raw numpy storage to torch
tensors on the device and back without changing a bit."""
import numpy as np
import torch

from oracle import mlx_affine as o

TORCH_DT = {o.BF16: torch.bfloat16, o.F16: torch.float16, o.F32: torch.float32}


def to_dev(raw: np.ndarray, dtype: int) -> torch.Tensor:
    if dtype == o.F32:
        return torch.from_numpy(np.ascontiguousarray(raw, dtype=np.float32)).cuda()
    t = torch.from_numpy(np.ascontiguousarray(raw, dtype=np.uint16).view(np.int16)).cuda()
    return t.view(TORCH_DT[dtype])


def u32_to_dev(raw: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(raw, dtype=np.uint32).view(np.int32)).cuda().view(torch.uint32)


def raw(t: torch.Tensor) -> np.ndarray:
    """torch tensor -> raw numpy storage (uint16 for 16-bit floats)."""
    t = t.detach().contiguous().cpu()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.uint32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


def to_f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.float64).cpu().numpy()
