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
# label_cost_active / augment_label_cost are shared by the launchers that take OTDD labels


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


def label_cost_active(label_x, label_y, label_cost_matrix, lambda_y: float) -> bool:
    """The reference's switch (kernels/sinkhorn_flashstyle_sqeuclid.py:1184-1189)."""
    return (label_x is not None and label_y is not None and label_cost_matrix is not None
            and lambda_y != 0.0)


def augment_label_cost(x: torch.Tensor, y: torch.Tensor, label_x: torch.Tensor,
                       label_y: torch.Tensor, label_cost_matrix: torch.Tensor,
                       lambda_x: float, lambda_y: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """OTDD label cost as V extra feature columns, so that the plain kernels apply.

    The reference adds ``- lambda_y*cs*W[label_i, label_j]`` to ``lambda_x*2cs*x_i.y_j`` with a
    per-element gather from W (kernels/sinkhorn_flashstyle_sqeuclid.py:546-560).  The same
    number is a dot product of augmented rows,
        x'_i = [lambda_x*x_i, -(lambda_y/2)*W[label_i, :]],   y'_j = [y_j, onehot(label_j)],
    since 2cs*x'_i.y'_j = lambda_x*2cs*x_i.y_j - lambda_y*cs*W[label_i, label_j]; the matrix
    cores then do the gather.  Validation and messages follow the reference (:1191-1210).
    Returns contiguous fp32 (x' [n, d+V], y' [m, d+V]).
    """
    n, m = x.shape[0], y.shape[0]
    if label_x.shape[0] != n:
        raise ValueError(f"label_x must have length n={n}, got {label_x.shape[0]}")
    if label_y.shape[0] != m:
        raise ValueError(f"label_y must have length m={m}, got {label_y.shape[0]}")
    if label_cost_matrix.ndim != 2:
        raise ValueError("label_cost_matrix must be 2D (V, V)")
    if label_cost_matrix.shape[0] != label_cost_matrix.shape[1]:
        raise ValueError("label_cost_matrix must be square (V, V)")
    V = label_cost_matrix.shape[0]
    if label_x.max() >= V or label_x.min() < 0:
        raise ValueError(f"label_x values must be in [0, {V}), got range "
                         f"[{label_x.min()}, {label_x.max()}]")
    if label_y.max() >= V or label_y.min() < 0:
        raise ValueError(f"label_y values must be in [0, {V}), got range "
                         f"[{label_y.min()}, {label_y.max()}]")
    lx = label_x.to(device=x.device, dtype=torch.long)
    ly = label_y.to(device=x.device, dtype=torch.long)
    W = label_cost_matrix.to(dtype=torch.float32, device=x.device)
    xa = torch.cat([float(lambda_x) * x.float(), (-0.5 * float(lambda_y)) * W[lx]], dim=1)
    ya = torch.cat([y.float(), torch.nn.functional.one_hot(ly, V).to(torch.float32)], dim=1)
    return xa.contiguous(), ya.contiguous()
