"""Scalar and small-vector helpers shared by the kernel launchers.

Mirrors the helper surface of the reference's ``kernels/_common.py:20-118``
(dampening, log_weights, max_diameter, epsilon_schedule, device validation).
The reference's Triton block-size / autotune tables have no counterpart here.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

__all__ = ["dampening", "log_weights", "max_diameter", "epsilon_schedule"]


def dampening(eps: float, rho: Optional[float]) -> float:
    """KL-relaxation factor 1/(1+eps/rho); 1.0 when the marginal is strict (rho=None)."""
    return 1.0 if rho is None else 1.0 / (1.0 + eps / rho)


def log_weights(w: torch.Tensor) -> torch.Tensor:
    """fp32 log(w) with non-positive weights mapped to -100000 (not -inf)."""
    w = w.float()
    return torch.where(w > 0, w.log(), torch.full_like(w, -100000.0))


def max_diameter(x: torch.Tensor, y: torch.Tensor) -> float:
    """Length of the diagonal of the joint bounding box of x and y (host float; syncs)."""
    xf, yf = x.float(), y.float()
    lo = torch.minimum(xf.amin(dim=0), yf.amin(dim=0))
    hi = torch.maximum(xf.amax(dim=0), yf.amax(dim=0))
    return (hi - lo).norm().item()


def epsilon_schedule(diameter: float, blur: float, scaling: float, p: float = 2.0) -> List[float]:
    """Geometric cooling diameter^p -> blur^p with ratio scaling^p (GeomLoss's schedule):
    [D^p] + [exp(e) for e in arange(p ln D, p ln blur, p ln scaling)] + [blur^p]."""
    if diameter <= 0:
        raise ValueError("diameter must be > 0.")
    if blur <= 0:
        raise ValueError("blur must be > 0.")
    if not (0.0 < scaling < 1.0):
        raise ValueError("scaling must be in (0, 1).")
    import numpy as np

    steps = np.arange(p * np.log(diameter), p * np.log(blur), p * np.log(scaling))
    return [diameter ** p] + [float(np.exp(e)) for e in steps] + [blur ** p]


def _validate_device(x: torch.Tensor, others: Sequence[Tuple[str, Optional[torch.Tensor]]]) -> None:
    """All tensors must live on x's (GPU) device."""
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    for name, t in others:
        if t is not None and t.device != x.device:
            raise ValueError(f"{name} must be on the same device as x ({x.device}), got {t.device}.")


def _f32c(t: torch.Tensor) -> torch.Tensor:
    """Contiguous fp32 view/copy of t (what every launcher hands to the C ABI)."""
    return t.contiguous().float()
