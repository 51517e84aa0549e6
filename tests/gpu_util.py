"""Helpers of the GPU parity tests: numpy <-> device tensors, synthetic projections, the tolerance measure."""
import numpy as np
import torch

MUL1, MCG = 0, 1


def dev_u16(a: np.ndarray) -> torch.Tensor:
    """uint16 host array -> int16 device tensor with the same bits (the kernels read the words, whatever their sign)."""
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def dev_f16_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.float16)).cuda()


def host_u16(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def make_x(rng: np.random.Generator, rows: int, in_f: int, dtype: torch.dtype, outliers: bool = False):
    """x [rows, in] ~ N(0, 1) representable in `dtype`: the device tensor and its values as f32."""
    x = rng.standard_normal((rows, in_f)).astype(np.float32)
    if outliers:
        mask = rng.random((rows, in_f)) < 0.01
        x = np.where(mask, x * 20.0, x).astype(np.float32)
    t = torch.from_numpy(x).to(dtype)
    return t.cuda(), t.to(torch.float32).numpy()


def to_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().to(torch.float32).cpu().numpy()


def bytes_of(t: torch.Tensor) -> bytes:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().tobytes()
