"""Dense numpy oracle for conjugate gradient and the Schur-complement HVP.

TEST INFRASTRUCTURE ONLY: the shipped package never imports this module.
Citations are into ``/root/reference/src/flash_sinkhorn`` (FS).

Pin status:
* conjugate_gradient ... numpy.linalg.solve on random SPD systems, iteration
  bookkeeping read off FS/cg.py:66-121
* hvp_x_from_potentials (balanced, full cost) ... golden vectors written from
  FS/testing/reference_hvp.py:33-152 (tests/golden/make_golden.py), plus
  finite differences of the oracle gradient through a converged fp64 solve
* hvp_x_from_potentials with rho_x/rho_y ... golden vectors from
  FS/testing/reference_hvp.py:155-356
* cost_scale=0.5 ... sqrt(2) rescaling identity against the full-cost golden
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional

import numpy as np

from oracle.sinkhorn_ref import log_weights, sqeuclid_cost

__all__ = ["CGResult", "conjugate_gradient", "geomloss_to_ott_potentials",
           "hvp_x_from_potentials", "inverse_hvp_x_from_potentials",
           "implicit_grad_x_from_potentials"]


@dataclass(frozen=True)
class CGResult:
    cg_converged: bool
    cg_iters: int
    cg_residual: float
    cg_initial_residual: float


def conjugate_gradient(matvec: Callable, b, *, x0=None, max_iter=300, rtol=1e-6, atol=1e-6,
                       preconditioner: Optional[Callable] = None, stabilise_every=0):
    """Textbook (P)CG (FS/cg.py:27-121): tol=max(atol, rtol*|r0|), stop when
    |r|<=tol, ``cg_iters=max_iter`` when not converged, break on p.Ap==0."""
    b = np.asarray(b)
    if stabilise_every < 0:
        raise ValueError("stabilise_every must be >= 0.")
    if x0 is None:
        x = np.zeros_like(b)
        r = b.copy()
    else:
        x = np.array(x0, copy=True)
        r = b - matvec(x)
    z = preconditioner(r) if preconditioner is not None else r
    p = z.copy()
    rz = float(r @ z)
    init = float(np.linalg.norm(r))
    tol = max(atol, rtol * init)
    for it in range(int(max_iter)):
        Ap = matvec(p)
        den = float(p @ Ap)
        if den == 0:
            break
        al = rz / den
        x = x + al * p
        r = r - al * Ap
        if stabilise_every and (it + 1) % stabilise_every == 0:
            r = b - matvec(x)
        res = float(np.linalg.norm(r))
        if res <= tol:
            return x, CGResult(True, it + 1, res, init)
        z = preconditioner(r) if preconditioner is not None else r
        rz_new = float(r @ z)
        p = z + (rz_new / rz) * p
        rz = rz_new
    return x, CGResult(False, int(max_iter), float(np.linalg.norm(r)), init)


def geomloss_to_ott_potentials(f, g, a, b, eps, dtype=np.float64):
    """f + eps*log a, g + eps*log b (FS/hvp.py:55-76)."""
    return (np.asarray(f, dtype) + eps * log_weights(a, dtype),
            np.asarray(g, dtype) + eps * log_weights(b, dtype))


def hvp_x_from_potentials(x, y, f_ott, g_ott, A, *, eps, rho_x=None, rho_y=None,
                          cost_scale=1.0, tau2=1e-5, max_cg_iter=300, cg_rtol=1e-6,
                          cg_atol=1e-6, cg_stabilise_every=0, preconditioner="none",
                          precond_terms=3, use_preconditioner=True, cg_x0=None,
                          dtype=np.float64):
    """Schur-complement Hessian-vector product w.r.t. x with a dense plan.

    Restates FS/hvp.py:282-623 (whose balanced full-cost dense twin is
    FS/testing/reference_hvp.py:33-152, the rho variant 155-356): OTT potentials,
    P = exp((f+g-C)/eps), marginal clamp (351-353), ``denom = diag_y + eps*tau2``
    only when both sides are balanced (393-396), un-preconditioned operator
    ``denom*z - P^T((P z)/diag_x)`` for mode "none" and ``z - Bz`` with
    ``rhs/denom`` otherwise (410-546).
    """
    x = np.asarray(x, dtype); y = np.asarray(y, dtype); A = np.asarray(A, dtype)
    cs = float(cost_scale)
    P = np.exp((np.asarray(f_ott, dtype)[:, None] + np.asarray(g_ott, dtype)[None, :]
                - sqeuclid_cost(x, y, cs, dtype)) / eps)
    a_hat = P.sum(axis=1)
    b_hat = P.sum(axis=0)
    balanced = rho_x is None and rho_y is None
    fx = 1.0 if rho_x is None else (rho_x + eps) / rho_x
    fy = 1.0 if rho_y is None else (rho_y + eps) / rho_y
    clamp = max(1e-12, eps * 1e-10)
    diag_x = fx * np.maximum(a_hat, clamp)
    diag_y = fy * np.maximum(b_hat, clamp)

    vec1 = (x * A).sum(axis=1)
    Py = P @ y
    x1 = 2.0 * cs * (a_hat * vec1 - (A * Py).sum(axis=1))
    PT_A = P.T @ A
    x2 = 2.0 * cs * (P.T @ vec1 - (y * PT_A).sum(axis=1))
    y1 = x1 / diag_x
    y2_raw = -(P.T @ y1) + x2
    denom = diag_y + eps * tau2 if balanced else diag_y

    def apply_B(z):
        return (P.T @ ((P @ z) / diag_x)) / denom

    mode = str(preconditioner).lower() if use_preconditioner else "none"
    if mode not in ("none", "neumann", "jacobi"):
        raise ValueError("preconditioner must be one of {'none','neumann','jacobi'}.")
    if int(precond_terms) < 0:
        raise ValueError("precond_terms must be >= 0.")
    if mode == "none":
        z, info = conjugate_gradient(
            lambda v: denom * v - P.T @ ((P @ v) / diag_x), y2_raw, x0=cg_x0,
            max_iter=max_cg_iter, rtol=cg_rtol, atol=cg_atol,
            stabilise_every=cg_stabilise_every)
    else:
        pre = None
        if mode == "neumann":
            def pre(v):
                out, cur = v, v
                for _ in range(int(precond_terms)):
                    cur = apply_B(cur)
                    out = out + cur
                return out
        z, info = conjugate_gradient(
            lambda v: v - apply_B(v), y2_raw / denom, x0=cg_x0, max_iter=max_cg_iter,
            rtol=cg_rtol, atol=cg_atol, preconditioner=pre,
            stabilise_every=cg_stabilise_every)

    z1 = y1 - (P @ z) / diag_x
    Py_z = P @ (y * z[:, None])
    RTz = 2.0 * cs * (x * (a_hat * z1)[:, None] - Py * z1[:, None]
                      + x * (P @ z)[:, None] - Py_z)
    Mat1 = 2.0 * cs * a_hat[:, None] * A
    Mat2 = (-4.0 * cs / eps) * x * (vec1 * a_hat)[:, None]
    Mat3 = (4.0 * cs / eps) * Py * vec1[:, None]
    Mat4 = (4.0 * cs / eps) * x * (Py * A).sum(axis=1)[:, None]
    Mat5 = (-4.0 * cs / eps) * ((P * (A @ y.T)) @ y)
    return RTz / eps + Mat1 + Mat2 + Mat3 + Mat4 + Mat5, info


def inverse_hvp_x_from_potentials(x, y, f_ott, g_ott, gr, *, eps, rho_x=None, rho_y=None,
                                  tau2=1e-5, dtype=np.float64):
    """z with H z = gr (FS/hvp.py:696-835), by assembling H column by column from
    ``hvp_x_from_potentials`` with a fully converged inner solve and a dense outer solve:
    what the reference's nested CG converges to.  Tiny inputs only (n*d HVPs)."""
    x = np.asarray(x, dtype)
    n, d = x.shape
    H = np.empty((n * d, n * d), dtype)
    for k in range(n * d):
        e = np.zeros(n * d, dtype)
        e[k] = 1.0
        col, _ = hvp_x_from_potentials(x, y, f_ott, g_ott, e.reshape(n, d), eps=eps, rho_x=rho_x,
                                       rho_y=rho_y, tau2=tau2, max_cg_iter=2000, cg_rtol=1e-13,
                                       cg_atol=1e-14, dtype=dtype)
        H[:, k] = col.reshape(-1)
    return np.linalg.solve(H, np.asarray(gr, dtype).reshape(-1)).reshape(n, d), H


def implicit_grad_x_from_potentials(x, y, f_hat, g_hat, grad_f, grad_g, *, eps, log_a=None,
                                    log_b=None, cost_scale=1.0, tau2=1e-5, dtype=np.float64):
    """Implicit-function-theorem gradient, restating FS/implicit_grad.py:113-242 with a dense
    plan and a dense solve of the regularised Schur system (:176-197); the 2/eps factor
    carries no cost_scale, as written (:240).  PARITY UNPINNED by any reference-held test."""
    x = np.asarray(x, dtype); y = np.asarray(y, dtype)
    n, m = x.shape[0], y.shape[0]
    la = np.full(n, -np.log(n), dtype) if log_a is None else np.asarray(log_a, dtype)
    lb = np.full(m, -np.log(m), dtype) if log_b is None else np.asarray(log_b, dtype)
    lg = (np.asarray(f_hat, dtype)[:, None] + np.asarray(g_hat, dtype)[None, :]
          + 2.0 * cost_scale * (x @ y.T)) / eps
    P = np.exp(lg + la[:, None] + lb[None, :])
    r, c = P.sum(axis=1), P.sum(axis=0)
    gf, gg = np.asarray(grad_f, dtype), np.asarray(grad_g, dtype)
    S = np.diag((c + eps * tau2) / eps) - (P.T @ (P / r[:, None])) / eps
    lam_g = np.linalg.solve(S, gg - P.T @ (gf / r))
    P_lam = P @ lam_g
    lam_f = eps * gf / r - P_lam / r
    return (2.0 / eps) * (lam_f[:, None] * (x * r[:, None] - P @ y)
                          + P_lam[:, None] * x - P @ (lam_g[:, None] * y))
