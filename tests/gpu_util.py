"""Helpers shared by the GPU parity tests."""

import numpy as np
import torch

DEV = torch.device("cuda", 0) if torch.cuda.is_available() else None


def to_np(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.uint32:
        return t.cpu().view(torch.int32).numpy().view(np.uint32)
    return t.cpu().numpy()


def rel_err(a: torch.Tensor, b: torch.Tensor) -> tuple[float, float]:
    """(max |a-b| / max |b|, ||a-b||_F / ||b||_F) in fp64."""
    a, b = a.double().cpu(), b.double().cpu()
    scale = float(b.abs().max())
    frob = float(b.norm())
    if scale == 0:
        return float((a - b).abs().max()), float((a - b).norm())
    return float((a - b).abs().max()) / scale, float((a - b).norm()) / frob
