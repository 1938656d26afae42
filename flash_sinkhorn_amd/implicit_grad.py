"""Gradient through the Sinkhorn fixed point by the implicit function theorem.

Host code over the streaming plan products, with the signatures of the reference's
``implicit_grad.py`` (``implicit_grad_x_from_potentials`` :36-242, ``implicit_grad_x``
:245-315).  At the fixed point the marginal residuals F = (P1 - a, P^T 1 - b) vanish; their
Jacobian in (f, g) is [[diag(r), P], [P^T, diag(c)]] / eps with r, c the row and column sums
of the plan.  The adjoint system J (lf, lg) = (grad_f, grad_g) is solved through its Schur
complement in lg with conjugate gradients, and
    dL/dx_i = (2/eps) [ lf_i (r_i x_i - (P y)_i) + (P lg)_i x_i - (P (lg * y))_i ].
The factor 2/eps carries no cost_scale, as in the reference (:240).
"""
from __future__ import annotations

import math
import warnings
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from flash_sinkhorn_amd.cg import conjugate_gradient
from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_sqeuclid import (
    apply_plan_mat_flashstyle,
    apply_plan_vec_flashstyle,
)

__all__ = ["ImplicitGradInfo", "implicit_grad_x_from_potentials", "implicit_grad_x"]


@dataclass(frozen=True)
class ImplicitGradInfo:
    cg_converged: bool
    cg_iters: int
    cg_residual: float


def implicit_grad_x_from_potentials(
    x: torch.Tensor, y: torch.Tensor, f_hat: torch.Tensor, g_hat: torch.Tensor,
    grad_f: torch.Tensor, grad_g: torch.Tensor, *, eps: float,
    log_a: Optional[torch.Tensor] = None, log_b: Optional[torch.Tensor] = None,
    cost_scale: float = 1.0, tau2: float = 1e-5, max_cg_iter: int = 100, cg_rtol: float = 1e-6,
    cg_atol: float = 1e-6, allow_tf32: bool = False, use_exp2: bool = True,
) -> Tuple[torch.Tensor, ImplicitGradInfo]:
    """dL/dx [n, d] for a loss with dL/df = grad_f, dL/dg = grad_g, at SHIFTED potentials
    f_hat = f - cs|x|^2, g_hat = g - cs|y|^2.  Missing log-weights mean uniform marginals."""
    if x.ndim != 2 or y.ndim != 2:
        raise ValueError("x, y must be 2D tensors.")
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    n, m = x.shape[0], y.shape[0]
    e = float(eps)
    if log_a is None:
        log_a = torch.full((n,), -math.log(n), device=x.device, dtype=torch.float32)
    if log_b is None:
        log_b = torch.full((m,), -math.log(m), device=x.device, dtype=torch.float32)
    kw = dict(eps=e, cost_scale=cost_scale, allow_tf32=allow_tf32, use_exp2=use_exp2)

    def P(v):   # [m] -> [n]
        return apply_plan_vec_flashstyle(x, y, f_hat, g_hat, log_a, log_b, v, axis=1, **kw)

    def PT(v):  # [n] -> [m]
        return apply_plan_vec_flashstyle(x, y, f_hat, g_hat, log_a, log_b, v, axis=0, **kw)

    def PM(mat, scale=None):
        return apply_plan_mat_flashstyle(x, y, f_hat, g_hat, log_a, log_b, mat, axis=1,
                                         scale=scale, **kw)

    r = P(torch.ones(m, device=x.device, dtype=torch.float32))
    c = PT(torch.ones(n, device=x.device, dtype=torch.float32))
    rhs = grad_g - PT(grad_f / r)
    diag = (c + e * tau2) / e
    lam_g, info = conjugate_gradient(lambda z: diag * z - PT(P(z) / r) / e, rhs,
                                     max_iter=max_cg_iter, rtol=cg_rtol, atol=cg_atol)
    P_lam = P(lam_g)
    lam_f = e * grad_f / r - P_lam / r
    yf = y.float()
    grad_x = (2.0 / e) * (lam_f[:, None] * (x * r[:, None] - PM(yf))
                          + P_lam[:, None] * x - PM(yf, scale=lam_g))
    return grad_x, ImplicitGradInfo(cg_converged=bool(info.cg_converged),
                                    cg_iters=int(info.cg_iters),
                                    cg_residual=float(info.cg_residual))


def implicit_grad_x(
    x: torch.Tensor, y: torch.Tensor, a: torch.Tensor, b: torch.Tensor, grad_f: torch.Tensor,
    grad_g: torch.Tensor, *, eps: float, cost_scale: float = 1.0, n_iters: int = 100,
    tau2: float = 1e-5, max_cg_iter: int = 100, cg_rtol: float = 1e-6, cg_atol: float = 1e-6,
    allow_tf32: bool = False, use_exp2: bool = True, autotune: bool = True,
    use_flashstyle: Optional[bool] = None,
) -> Tuple[torch.Tensor, ImplicitGradInfo]:
    """Solve Sinkhorn at fixed eps (n_iters symmetric iterations with the last extrapolation),
    then ``implicit_grad_x_from_potentials``."""
    if use_flashstyle is not None and not use_flashstyle:
        warnings.warn("use_flashstyle=False is deprecated. FlashSinkhorn is now the only backend.",
                      DeprecationWarning, stacklevel=2)
    from flash_sinkhorn_amd.sinkhorn_solvers import sinkhorn_flashstyle_symmetric

    f, g = sinkhorn_flashstyle_symmetric(
        x, y, a, b, use_epsilon_scaling=False, eps=eps, cost_scale=cost_scale, n_iters=n_iters,
        last_extrapolation=True, allow_tf32=allow_tf32, use_exp2=use_exp2)
    f_hat = f - cost_scale * (x.float() ** 2).sum(dim=1)
    g_hat = g - cost_scale * (y.float() ** 2).sum(dim=1)
    return implicit_grad_x_from_potentials(
        x, y, f_hat, g_hat, grad_f, grad_g, eps=eps, log_a=torch.log(a.clamp(min=1e-20)),
        log_b=torch.log(b.clamp(min=1e-20)), cost_scale=cost_scale, tau2=tau2,
        max_cg_iter=max_cg_iter, cg_rtol=cg_rtol, cg_atol=cg_atol, allow_tf32=allow_tf32,
        use_exp2=use_exp2)
