"""Hessian-vector product of the Sinkhorn cost w.r.t. x, plan never materialised.

Entry points and conventions of the reference's ``hvp.py``: ``HvpInfo`` (:44-52),
``geomloss_to_ott_potentials`` (:55-76), ``sinkhorn_prelast_potentials_sqeuclid``
(:103-161), ``hvp_x_sqeuclid_from_potentials`` (:164-623), ``hvp_x_sqeuclid``
(:626-693).  The product is the Schur-complement form

    H A = R^T (H*)^-1 R A / eps + E A,

with every plan product done by the streaming HIP kernels: two matrix products
and four vector products for the right-hand side, two vector products per CG
iteration on ``denom*z - P^T((P z)/diag_x)``, then one scaled matrix product, and
the Mat5 kernel.  The alternative CG drivers of the reference (dense cached plan,
torch.compile, batched, fused two-phase matvec) are not built.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.cg import conjugate_gradient, conjugate_gradient_device
from flash_sinkhorn_amd.kernels._common import log_weights
from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_sqeuclid import (
    apply_plan_mat_flashstyle, apply_plan_vec_flashstyle, mat5_sqeuclid,
)
from flash_sinkhorn_amd.sinkhorn_solvers import sinkhorn_flashstyle_symmetric

__all__ = ["HvpInfo", "geomloss_to_ott_potentials", "ott_to_geomloss_potentials",
           "sinkhorn_prelast_potentials_sqeuclid", "hvp_x_sqeuclid",
           "hvp_x_sqeuclid_from_potentials", "inverse_hvp_x_sqeuclid_from_potentials"]


@dataclass(frozen=True)
class HvpInfo:
    cg_converged: bool
    cg_iters: int
    cg_residual: float
    cg_initial_residual: float
    converged_lambda: float = 0.0
    hit_neg_curv: bool = False
    diagnostic_msg: str = ""


def geomloss_to_ott_potentials(f, g, a, b, *, eps: float):
    """(f + eps*log a, g + eps*log b): from P = a b exp((f+g-C)/eps) to P = exp((f+g-C)/eps)."""
    e = float(eps)
    return f.float() + e * log_weights(a), g.float() + e * log_weights(b)


def ott_to_geomloss_potentials(f_hat, g_hat, a, b, *, eps: float):
    e = float(eps)
    return f_hat.float() - e * log_weights(a), g_hat.float() - e * log_weights(b)


def sinkhorn_prelast_potentials_sqeuclid(
    x, y, a, b, *, eps_list: Sequence[float], allow_tf32: bool = False, use_exp2: bool = True,
    autotune: bool = True, block_m=None, block_n=None, block_k=None, num_warps=None,
    num_stages: int = 2, use_flashstyle: Optional[bool] = None, cost_scale: float = 1.0,
    rho_x: Optional[float] = None, rho_y: Optional[float] = None,
):
    """Pre-extrapolation potentials of the symmetric solver run on ``eps_list``."""
    _, _, f_grad, g_grad = sinkhorn_flashstyle_symmetric(
        x, y, a, b, use_epsilon_scaling=False, last_extrapolation=True, allow_tf32=allow_tf32,
        use_exp2=use_exp2, eps_list=eps_list, return_prelast=True, cost_scale=cost_scale,
        rho_x=rho_x, rho_y=rho_y)
    return f_grad, g_grad


def hvp_x_sqeuclid_from_potentials(
    x: torch.Tensor, y: torch.Tensor, f_hat: torch.Tensor, g_hat: torch.Tensor, A: torch.Tensor, *,
    eps: float, rho_x: Optional[float] = None, rho_y: Optional[float] = None,
    cost_scale: float = 1.0, lambda_indef: float = 1.0, return_components: bool = False,
    tau2: float = 1e-5, max_cg_iter: int = 300, cg_rtol: float = 1e-6, cg_atol: float = 1e-6,
    cg_stabilise_every: int = 0, preconditioner: str = "none", precond_terms: int = 3,
    use_preconditioner: bool = True, allow_tf32: bool = False, use_exp2: bool = True,
    block_m=None, block_n=None, block_k=None, num_warps: int = 4, num_stages: int = 2,
    use_fused_matvec: bool = False, use_batched_cg: bool = False, use_compiled_cg: bool = False,
    use_dense_cg: bool = False, autotune: bool = True, cg_x0: Optional[torch.Tensor] = None,
):
    """H @ A for OTT-convention potentials (f_hat, g_hat); returns (hvp [n,d], HvpInfo).

    Balanced problems regularise the Schur complement with ``eps*tau2``; with
    rho_x / rho_y the diagonal blocks are scaled by (rho+eps)/rho and no
    regularisation is added.  ``preconditioner``: "none" solves
    ``denom*z - P^T((Pz)/diag_x) = rhs``; "neumann"/"jacobi" solve ``z - Bz = rhs/denom``
    (Neumann adds ``precond_terms`` terms of the series as M^-1).
    """
    if x.ndim != 2 or y.ndim != 2 or A.ndim != 2:
        raise ValueError("x,y,A must be 2D tensors.")
    if not x.is_cuda or not y.is_cuda or not f_hat.is_cuda or not g_hat.is_cuda:
        raise ValueError("hvp_x_sqeuclid_from_potentials requires CUDA tensors.")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2 or A.shape != (n, d):
        raise ValueError("Shapes must satisfy x:(n,d), y:(m,d), A:(n,d).")
    if use_dense_cg or use_compiled_cg or use_batched_cg:
        raise NotImplementedError(
            "only the streaming CG driver is built (dense/compiled/batched drivers are not)")
    mode = str(preconditioner).lower() if use_preconditioner else "none"
    if mode not in ("none", "neumann", "jacobi"):
        raise ValueError("preconditioner must be one of {'none','neumann','jacobi'}.")
    n_terms = int(precond_terms)
    if n_terms < 0:
        raise ValueError("precond_terms must be >= 0.")

    e = float(eps)
    cs = float(cost_scale)
    xf, yf, Af = x.float().contiguous(), y.float().contiguous(), A.float().contiguous()
    x_sq = (xf * xf).sum(dim=1).contiguous()
    y_sq = (yf * yf).sum(dim=1).contiguous()

    # Shifted potentials with a uniform log-weight gauge (any constant cancels between the
    # conversion and the kernels' own +log a, +log b).
    log_a = torch.full((n,), -math.log(n), device=x.device, dtype=torch.float32)
    log_b = torch.full((m,), -math.log(m), device=x.device, dtype=torch.float32)
    f_sh = (f_hat.float() - e * log_a - cs * x_sq).contiguous()
    g_sh = (g_hat.float() - e * log_b - cs * y_sq).contiguous()
    kw = dict(eps=e, cost_scale=cs, allow_tf32=allow_tf32, use_exp2=use_exp2)

    def P(v):   # [m] -> [n]
        return apply_plan_vec_flashstyle(xf, yf, f_sh, g_sh, log_a, log_b, v, axis=1, **kw)

    def PT(v):  # [n] -> [m]
        return apply_plan_vec_flashstyle(xf, yf, f_sh, g_sh, log_a, log_b, v, axis=0, **kw)

    def Pmat(V, scale=None):
        return apply_plan_mat_flashstyle(xf, yf, f_sh, g_sh, log_a, log_b, V, axis=1,
                                         scale=scale, **kw)

    row_mass = P(torch.ones((m,), device=x.device, dtype=torch.float32))
    col_mass = PT(torch.ones((n,), device=x.device, dtype=torch.float32))
    balanced = rho_x is None and rho_y is None
    fac_x = 1.0 if rho_x is None else (float(rho_x) + e) / float(rho_x)
    fac_y = 1.0 if rho_y is None else (float(rho_y) + e) / float(rho_y)
    floor = max(1e-12, e * 1e-10)
    diag_x = fac_x * row_mass.clamp(min=floor)
    diag_y = fac_y * col_mass.clamp(min=floor)
    denom = diag_y + e * float(tau2) if balanced else diag_y

    xa = (xf * Af).sum(dim=1)
    Py = Pmat(yf)
    r1 = (2.0 * cs) * (row_mass * xa - (Af * Py).sum(dim=1))
    PtA = apply_plan_mat_flashstyle(xf, yf, f_sh, g_sh, log_a, log_b, Af, axis=0, **kw)
    r2 = (2.0 * cs) * (PT(xa) - (yf * PtA).sum(dim=1))
    y1 = r1 / diag_x
    rhs = r2 - PT(y1)

    def B(v):
        return PT(P(v) / diag_x) / denom

    if mode == "none" and cg_x0 is None and not cg_stabilise_every:
        # CG bookkeeping on the device; small problems look at the state every few iterations
        # (their iterations are launch bound), large ones after each (a wasted matvec costs more
        # than a read-back)
        from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_fused_sqeuclid import (
            _schur_matvec_raw)
        inv_diag_x = (1.0 / diag_x).contiguous()
        denom_c = denom.contiguous()
        piz_buf = torch.empty((n,), device=x.device, dtype=torch.float32)
        schur_ws = _lib.workspace(_lib.OP_APPLY_VEC, n, m, d, x.device)

        def schur(v):  # denom * v - P^T((P v) / diag_x): two launches, factors in the epilogues
            return _schur_matvec_raw(xf, yf, f_sh, g_sh, log_a, log_b, v, inv_diag_x, denom_c,
                                     eps=e, cost_scale=cs, allow_tf32=allow_tf32,
                                     use_exp2=use_exp2, piz=piz_buf, workspace=schur_ws)[0]

        z, cg = conjugate_gradient_device(
            schur, rhs, max_iter=max_cg_iter, rtol=cg_rtol, atol=cg_atol,
            check_every=4 if float(n) * float(m) * float(d) < 2.0e9 else 1)
    elif mode == "none":
        z, cg = conjugate_gradient(
            lambda v: denom * v - PT(P(v) / diag_x), rhs, x0=cg_x0, max_iter=max_cg_iter,
            rtol=cg_rtol, atol=cg_atol, preconditioner=None, stabilise_every=cg_stabilise_every)
    else:
        series = None
        if mode == "neumann":
            def series(v):
                total, term = v, v
                for _ in range(n_terms):
                    term = B(term)
                    total = total + term
                return total
        z, cg = conjugate_gradient(
            lambda v: v - B(v), rhs / denom, x0=cg_x0, max_iter=max_cg_iter, rtol=cg_rtol,
            atol=cg_atol, preconditioner=series, stabilise_every=cg_stabilise_every)

    Pz = P(z)
    z1 = y1 - Pz / diag_x
    Py_z = Pmat(yf, scale=z)
    RTz = (2.0 * cs) * (xf * (row_mass * z1 + Pz)[:, None] - Py * z1[:, None] - Py_z)

    c4 = 4.0 * cs / e
    psd = RTz / e + (2.0 * cs) * row_mass[:, None] * Af
    ya = (Py * Af).sum(dim=1)
    indef = (c4 * (ya - xa * row_mass))[:, None] * xf + c4 * Py * xa[:, None]
    indef = indef + mat5_sqeuclid(xf, yf, f_hat, g_hat, Af, eps=e, cost_scale=cs, x2=x_sq,
                                  y2=y_sq, allow_tf32=allow_tf32, use_exp2=use_exp2)

    info = HvpInfo(bool(cg.cg_converged), int(cg.cg_iters), float(cg.cg_residual),
                   float(cg.cg_initial_residual))
    if return_components:
        return psd, indef, info
    return (psd + indef if lambda_indef == 1.0 else psd + lambda_indef * indef), info


def hvp_x_sqeuclid(
    x, y, a, b, A, *, eps_list: Sequence[float], tau2: float = 1e-5, max_cg_iter: int = 300,
    cg_rtol: float = 1e-6, cg_atol: float = 1e-6, cg_stabilise_every: int = 0,
    preconditioner: str = "none", precond_terms: int = 3, use_preconditioner: bool = True,
    allow_tf32: bool = False, use_exp2: bool = True, autotune: bool = True, block_m=None,
    block_n=None, block_k=None, num_warps=None, num_stages: int = 2,
):
    """Solve for the pre-extrapolation potentials on ``eps_list``, then H @ A."""
    eps = float(eps_list[-1])
    f_grad, g_grad = sinkhorn_prelast_potentials_sqeuclid(
        x, y, a, b, eps_list=eps_list, allow_tf32=allow_tf32, use_exp2=use_exp2)
    f_hat, g_hat = geomloss_to_ott_potentials(f_grad, g_grad, a, b, eps=eps)
    return hvp_x_sqeuclid_from_potentials(
        x, y, f_hat, g_hat, A, eps=eps, tau2=tau2, max_cg_iter=max_cg_iter, cg_rtol=cg_rtol,
        cg_atol=cg_atol, cg_stabilise_every=cg_stabilise_every, preconditioner=preconditioner,
        precond_terms=precond_terms, use_preconditioner=use_preconditioner,
        allow_tf32=allow_tf32, use_exp2=use_exp2)


def inverse_hvp_x_sqeuclid_from_potentials(
    x, y, f_hat, g_hat, gr, *, eps: float, rho_x: Optional[float] = None,
    rho_y: Optional[float] = None, tau2: float = 1e-5, max_outer_iter: int = 100,
    outer_rtol: float = 1e-6, outer_atol: float = 1e-6, max_inner_iter: int = 100,
    inner_rtol: float = 1e-8, inner_atol: float = 1e-8, cg_stabilise_every: int = 0,
    preconditioner: str = "none", precond_terms: int = 3, use_preconditioner: bool = True,
    allow_tf32: bool = False, use_exp2: bool = True, block_m=None, block_n=None, block_k=None,
    num_warps: int = 4, num_stages: int = 2,
) -> Tuple[torch.Tensor, HvpInfo]:
    """z with H z = gr, H the Hessian w.r.t. x at the given OTT potentials: an outer CG on the
    flattened (n*d) vector whose matvec is ``hvp_x_sqeuclid_from_potentials`` (itself an inner
    CG on the Schur complement).  Same signature and bookkeeping as the reference's
    ``hvp.py:696-835``; ``HvpInfo`` reports the OUTER solve."""
    if x.ndim != 2 or y.ndim != 2 or gr.ndim != 2:
        raise ValueError("x, y, gr must be 2D tensors.")
    if not x.is_cuda or not y.is_cuda or not f_hat.is_cuda or not g_hat.is_cuda:
        raise ValueError("inverse_hvp_x_sqeuclid_from_potentials requires CUDA tensors.")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2 or gr.shape != (n, d):
        raise ValueError("Shapes must satisfy x:(n,d), y:(m,d), gr:(n,d).")

    def matvec(v_flat: torch.Tensor) -> torch.Tensor:
        out, _ = hvp_x_sqeuclid_from_potentials(
            x, y, f_hat, g_hat, v_flat.reshape(n, d), eps=eps, rho_x=rho_x, rho_y=rho_y,
            tau2=tau2, max_cg_iter=max_inner_iter, cg_rtol=inner_rtol, cg_atol=inner_atol,
            cg_stabilise_every=cg_stabilise_every, preconditioner=preconditioner,
            precond_terms=precond_terms, use_preconditioner=use_preconditioner,
            allow_tf32=allow_tf32, use_exp2=use_exp2)
        return out.reshape(-1)

    z, info = conjugate_gradient(matvec, gr.float().reshape(-1), max_iter=max_outer_iter,
                                 rtol=outer_rtol, atol=outer_atol, preconditioner=None,
                                 stabilise_every=cg_stabilise_every)
    return z.reshape(n, d), HvpInfo(
        cg_converged=bool(info.cg_converged), cg_iters=int(info.cg_iters),
        cg_residual=float(info.cg_residual), cg_initial_residual=float(info.cg_initial_residual))
