"""Hard c-transform for the squared-Euclidean cost and its semi-dual objective.

Public names and behaviour of the reference's ``c_transform.py``:
    c^psi(x_i) = min_j [cost_scale*|x_i - y_j|^2 - psi_j],   j*(i) = argmin_j [same]
    L(x, psi)  = sum_i a_i c^psi(x_i) + sum_j b_j psi_j
``c_transform_fwd`` (:32-112) returns values and argmin without autograd;
``c_transform_cost`` (:177-241) is differentiable in x and psi by Danskin's theorem
(:115-174): dL/dx_i = a_i*2*cost_scale*(x_i - y_{j*(i)}),  dL/dpsi_j = b_j - sum_{i: j*(i)=j} a_i.
Gradients with respect to y are not provided, as in the reference.
"""
from __future__ import annotations

from typing import Optional

import torch

from flash_sinkhorn_amd.kernels._common import _validate_device
from flash_sinkhorn_amd.kernels.c_transform_sqeuclid import c_transform_kernel

__all__ = ["c_transform_fwd", "c_transform_cost"]


def c_transform_fwd(x: torch.Tensor, y: torch.Tensor, psi: torch.Tensor, *,
                    cost_scale: float = 1.0, allow_tf32: bool = True, autotune: bool = True,
                    **kernel_kwargs) -> tuple[torch.Tensor, torch.Tensor]:
    """(c_values [n] float32, argmin_idx [n] int64), both detached."""
    if x.ndim != 2:
        raise ValueError(f"x must be 2D [n, d], got shape {x.shape}")
    if y.ndim != 2:
        raise ValueError(f"y must be 2D [m, d], got shape {y.shape}")
    if psi.ndim != 1:
        raise ValueError(f"psi must be 1D [m], got shape {psi.shape}")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError(f"x and y must have same feature dim, got {d} vs {d2}")
    if psi.shape[0] != m:
        raise ValueError(f"psi must have length {m}, got {psi.shape[0]}")
    if m == 0:
        raise ValueError("m must be > 0")
    if not x.is_cuda:
        raise ValueError("x must be a CUDA tensor")
    _validate_device(x, [("y", y), ("psi", psi)])
    if y.requires_grad:
        raise NotImplementedError("grad_y not supported for c_transform_fwd. "
                                  "Detach y or use a solver that supports grad_y.")
    with torch.no_grad():
        xf, yf = x.float(), y.float()
        bias = cost_scale * (yf * yf).sum(dim=1) - psi.float()
        inner, idx = c_transform_kernel(xf, yf, bias, cost_scale=cost_scale,
                                        allow_tf32=allow_tf32, autotune=autotune,
                                        **kernel_kwargs)
        values = cost_scale * (xf * xf).sum(dim=1) + inner
    return values, idx


class _CTransformCostFunction(torch.autograd.Function):
    """Semi-dual objective with the Danskin gradients at the minimiser j*(i)."""

    @staticmethod
    def forward(ctx, x, y, psi, cost_scale, allow_tf32, autotune, a, b):
        values, idx = c_transform_fwd(x, y, psi, cost_scale=cost_scale, allow_tf32=allow_tf32,
                                      autotune=autotune)
        ctx.save_for_backward(x, y, idx, a, b)
        ctx.cost_scale = cost_scale
        return (a * values).sum() + (b * psi.float()).sum()

    @staticmethod
    def backward(ctx, grad_output):
        x, y, idx, a, b = ctx.saved_tensors
        if ctx.needs_input_grad[1]:
            raise NotImplementedError("grad_y not implemented for c_transform_cost. "
                                      "Detach y before passing to c_transform_cost.")
        grad_x = grad_psi = None
        if ctx.needs_input_grad[0]:
            matched = y.float()[idx]
            grad_x = grad_output * (2.0 * ctx.cost_scale * a).unsqueeze(1) * (x.float() - matched)
        if ctx.needs_input_grad[2]:
            assigned = torch.zeros(y.shape[0], device=a.device, dtype=torch.float32)
            assigned.scatter_add_(0, idx, a)
            grad_psi = grad_output * (b - assigned)
        return grad_x, None, grad_psi, None, None, None, None, None


def c_transform_cost(x: torch.Tensor, y: torch.Tensor, psi: torch.Tensor, *,
                     cost_scale: float = 1.0, allow_tf32: bool = True, autotune: bool = True,
                     a: Optional[torch.Tensor] = None,
                     b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Scalar L(x, psi); weights default to uniform and must not require grad."""
    n, m = x.shape[0], y.shape[0]
    if a is None:
        a = torch.full((n,), 1.0 / n, device=x.device, dtype=torch.float32)
    if b is None:
        b = torch.full((m,), 1.0 / m, device=y.device, dtype=torch.float32)
    if a.shape != (n,):
        raise ValueError(f"a must have shape ({n},), got {a.shape}")
    if b.shape != (m,):
        raise ValueError(f"b must have shape ({m},), got {b.shape}")
    _validate_device(x, [("a", a), ("b", b)])
    if a.requires_grad:
        raise ValueError("a must not require grad (weights are non-differentiable)")
    if b.requires_grad:
        raise ValueError("b must not require grad (weights are non-differentiable)")
    return _CTransformCostFunction.apply(x, y, psi, cost_scale, allow_tf32, autotune, a.float(),
                                         b.float())
