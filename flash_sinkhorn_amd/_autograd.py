"""Autograd wiring of the Sinkhorn cost: analytic gradient, HVP as double backward.

Mirrors the reference's ``_autograd.py``: ``_SinkhornConfig`` (:33-76),
``_SinkhornCostFn`` (forward = solver + cost formula :306-455, backward = gradient
operator :457-519) and ``_SinkhornGradFn`` (forward = gradient kernel :91-181,
backward = Hessian-vector product w.r.t. x :183-283).  No backpropagation through
the Sinkhorn iterations: the gradient is taken at the pre-extrapolation potentials.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from flash_sinkhorn_amd.hvp import geomloss_to_ott_potentials, hvp_x_sqeuclid_from_potentials
from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
    sinkhorn_geomloss_online_grad_sqeuclid,
)
from flash_sinkhorn_amd.sinkhorn_solvers import (
    sinkhorn_flashstyle_alternating, sinkhorn_flashstyle_symmetric,
)


@dataclass(frozen=True)
class _SinkhornConfig:
    """Immutable snapshot of a SamplesLoss instance's settings."""
    backend: str
    blur: float
    scaling: float
    use_epsilon_scaling: bool
    eps: Optional[float]
    n_iters: Optional[int]
    cost_scale: float
    rho_x: Optional[float]
    rho_y: Optional[float]
    last_extrapolation: bool
    allow_tf32: bool
    use_exp2: bool
    autotune: bool
    block_m: Optional[int]
    block_n: Optional[int]
    block_k: Optional[int]
    num_warps: Optional[int]
    num_stages: int
    hvp_tau2: float
    hvp_max_cg_iter: int
    hvp_cg_rtol: float
    hvp_cg_atol: float
    hvp_cg_stabilise_every: int
    hvp_preconditioner: str
    hvp_precond_terms: int
    hvp_use_preconditioner: bool
    lambda_x: float
    lambda_y: float
    threshold: Optional[float]
    inner_iterations: int


class _SinkhornGradFn(torch.autograd.Function):
    """(grad_x, grad_y) of the cost at fixed potentials; differentiable once more in x."""

    @staticmethod
    def forward(ctx, x, y, a, b, f_grad, g_grad, grad_scale, eps: float,
                config: _SinkhornConfig, compute_grad_x: bool, compute_grad_y: bool,
                label_x=None, label_y=None, label_cost_matrix=None, seed_keys=None):
        gx, gy = sinkhorn_geomloss_online_grad_sqeuclid(
            x, y, a, b, f_grad, g_grad, eps=float(eps), allow_tf32=config.allow_tf32,
            use_exp2=config.use_exp2, grad_scale=grad_scale,
            compute_grad_x=bool(compute_grad_x), compute_grad_y=bool(compute_grad_y),
            cost_scale=config.cost_scale, label_x=label_x, label_y=label_y,
            label_cost_matrix=label_cost_matrix, lambda_x=config.lambda_x,
            lambda_y=config.lambda_y, _seed_keys=seed_keys)
        ctx.save_for_backward(x, y, a, b, f_grad, g_grad, grad_scale)
        ctx.eps = float(eps)
        ctx.config = config
        ctx.use_label_cost = (label_x is not None and label_y is not None
                              and label_cost_matrix is not None and config.lambda_y != 0.0)
        return gx, gy

    @staticmethod
    def backward(ctx, grad_grad_x, grad_grad_y):
        x, y, a, b, f_grad, g_grad, grad_scale = ctx.saved_tensors
        cfg = ctx.config
        if grad_grad_y is not None:
            raise NotImplementedError("Double backward w.r.t y is not implemented yet.")
        if ctx.use_label_cost:
            raise NotImplementedError(
                "Double backward (HVP) is not supported with OTDD label-augmented cost.")
        out_x = None
        if grad_grad_x is not None:
            if grad_grad_x.shape != x.shape:
                raise ValueError("grad_grad_x must have the same shape as x.")
            if not grad_grad_x.is_cuda:
                raise ValueError("grad_grad_x must be a CUDA tensor.")
            with torch.no_grad():
                f_ott, g_ott = geomloss_to_ott_potentials(f_grad, g_grad, a, b, eps=ctx.eps)
                hvp, _ = hvp_x_sqeuclid_from_potentials(
                    x, y, f_ott, g_ott, grad_grad_x, eps=ctx.eps, rho_x=cfg.rho_x,
                    rho_y=cfg.rho_y, cost_scale=cfg.cost_scale, tau2=cfg.hvp_tau2,
                    max_cg_iter=cfg.hvp_max_cg_iter, cg_rtol=cfg.hvp_cg_rtol,
                    cg_atol=cfg.hvp_cg_atol, cg_stabilise_every=cfg.hvp_cg_stabilise_every,
                    preconditioner=cfg.hvp_preconditioner, precond_terms=cfg.hvp_precond_terms,
                    use_preconditioner=cfg.hvp_use_preconditioner,
                    allow_tf32=False,  # second order needs full fp32 operands
                    use_exp2=cfg.use_exp2)
                out_x = hvp * grad_scale
        return (out_x,) + (None,) * 14


class _SinkhornCostFn(torch.autograd.Function):
    """OT cost from one Sinkhorn solve; backward is the analytic gradient operator."""

    @staticmethod
    def forward(ctx, x, y, a, b, eps_list: Tuple[float, ...], config: _SinkhornConfig,
                label_x, label_y, label_cost_matrix, presolved=None):
        """``presolved``: the tuple ``sinkhorn_flashstyle_symmetric`` would return for this
        problem (with ``return_prelast=config.last_extrapolation``), when the caller has already
        run the solve (the two self terms of a debiased loss are solved together)."""
        eps_last = float(eps_list[-1])
        seed_keys = None
        if presolved is not None:
            if config.last_extrapolation:
                f_cost, g_cost, f_grad, g_grad = presolved
            else:
                f_cost, g_cost = presolved
                f_grad, g_grad = f_cost, g_cost
            balanced_formula = config.rho_x is None or config.rho_y is None
        elif config.backend == "alternating":
            f_cost, g_cost = sinkhorn_flashstyle_alternating(
                x, y, a, b, eps=eps_last, n_iters=len(eps_list), cost_scale=config.cost_scale,
                rho_x=config.rho_x, rho_y=config.rho_y, allow_tf32=config.allow_tf32,
                use_exp2=config.use_exp2)
            f_grad, g_grad = f_cost, g_cost
            balanced_formula = True
        else:
            info = {}
            out = sinkhorn_flashstyle_symmetric(
                x, y, a, b, solve_info=info, blur=config.blur, scaling=config.scaling,
                use_epsilon_scaling=config.use_epsilon_scaling, eps=config.eps,
                n_iters=config.n_iters, allow_tf32=config.allow_tf32, use_exp2=config.use_exp2,
                cost_scale=config.cost_scale, rho_x=config.rho_x, rho_y=config.rho_y,
                last_extrapolation=config.last_extrapolation,
                return_prelast=config.last_extrapolation, threshold=config.threshold,
                check_every=config.inner_iterations, label_x=label_x, label_y=label_y,
                label_cost_matrix=label_cost_matrix, lambda_x=config.lambda_x,
                lambda_y=config.lambda_y)
            if config.last_extrapolation:
                f_cost, g_cost, f_grad, g_grad = out
            else:
                f_cost, g_cost = out
                f_grad, g_grad = f_cost, g_cost
            # <a,f>+<b,g> unless BOTH marginals are relaxed
            balanced_formula = config.rho_x is None or config.rho_y is None
            # the keys behind the rows' largest logits, where the solve kept them: a hint from
            # which the gradient's sweep recognises the tiles that cannot matter
            prep = info.get("prepared")
            if prep is not None and info.get("coarse"):
                kx, ky = prep.best_keys(0), prep.best_keys(1)
                if kx is not None and ky is not None:
                    seed_keys = (kx.clone(), ky.clone())

        ctx.save_for_backward(x, y, a, b, f_cost, g_cost, f_grad, g_grad)
        ctx.eps = eps_last
        ctx.config = config
        ctx.seed_keys = seed_keys
        labelled = config.backend != "alternating"  # the alternating backend takes no labels
        ctx.labels = (label_x, label_y, label_cost_matrix) if labelled else (None, None, None)
        if balanced_formula:
            return (a * f_cost).sum() + (b * g_cost).sum()
        wx = config.rho_x + eps_last / 2
        wy = config.rho_y + eps_last / 2
        return (wx * (a * (1 - (-f_cost / config.rho_x).exp())).sum()
                + wy * (b * (1 - (-g_cost / config.rho_y).exp())).sum())

    @staticmethod
    def backward(ctx, grad_out):
        x, y, a, b, f_cost, g_cost, f_grad, g_grad = ctx.saved_tensors
        grad_x = grad_y = grad_a = grad_b = None
        if x.requires_grad or y.requires_grad:
            gx, gy = _SinkhornGradFn.apply(x, y, a, b, f_grad, g_grad, grad_out, ctx.eps,
                                           ctx.config, x.requires_grad, y.requires_grad,
                                           *ctx.labels, ctx.seed_keys)
            grad_x = gx if x.requires_grad else None
            grad_y = gy if y.requires_grad else None
        if a.requires_grad:
            grad_a = grad_out * f_cost
        if b.requires_grad:
            grad_b = grad_out * g_cost
        return grad_x, grad_y, grad_a, grad_b, None, None, None, None, None, None
