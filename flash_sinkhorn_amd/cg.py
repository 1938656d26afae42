"""Conjugate gradient on device vectors (host-driven loop).

``conjugate_gradient`` and ``CGInfo`` follow the reference's ``cg.py:19-121``:
tolerance ``max(atol, rtol*|r0|)``, stop as soon as ``|r| <= tol``, report
``cg_iters = max_iter`` when the loop ends without converging, and leave the loop
when the curvature ``p.Ap`` is exactly zero.  One host read-back per iteration
(the residual norm) decides whether to stop.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional, Tuple

import torch

__all__ = ["CGInfo", "conjugate_gradient", "conjugate_gradient_device"]


@dataclass(frozen=True)
class CGInfo:
    cg_converged: bool
    cg_iters: int
    cg_residual: float
    cg_initial_residual: float


def _norm(v: torch.Tensor) -> float:
    return float(torch.linalg.norm(v).detach().cpu())


def conjugate_gradient(
    matvec: Callable[[torch.Tensor], torch.Tensor],
    b: torch.Tensor,
    *,
    x0: Optional[torch.Tensor] = None,
    max_iter: int = 300,
    rtol: float = 1e-6,
    atol: float = 1e-6,
    preconditioner: Optional[Callable[[torch.Tensor], torch.Tensor]] = None,
    stabilise_every: int = 0,
) -> Tuple[torch.Tensor, CGInfo]:
    """Solve ``A x = b`` for symmetric positive definite ``A`` given as ``matvec``.

    ``x0`` warm-starts the iteration; ``preconditioner`` applies M^-1;
    ``stabilise_every=k`` recomputes the true residual every k iterations.
    """
    every = int(stabilise_every)
    if every < 0:
        raise ValueError("stabilise_every must be >= 0.")
    apply_m = preconditioner if preconditioner is not None else (lambda r: r)

    if x0 is None:
        sol = torch.zeros_like(b)
        res = b.clone()
    else:
        sol = x0.clone()
        res = b - matvec(sol)
    z = apply_m(res)
    direction = z.clone()
    rz = torch.dot(res, z)
    r0 = _norm(res)
    tol = max(atol, rtol * r0)

    for k in range(int(max_iter)):
        a_dir = matvec(direction)
        curvature = torch.dot(direction, a_dir)
        if curvature.abs() == 0:
            break
        step = rz / curvature
        sol = sol + step * direction
        res = res - step * a_dir
        if every and (k + 1) % every == 0:
            res = b - matvec(sol)
        rnorm = _norm(res)
        if rnorm <= tol:
            return sol, CGInfo(True, k + 1, rnorm, r0)
        z = apply_m(res)
        rz_next = torch.dot(res, z)
        direction = z + (rz_next / rz) * direction
        rz = rz_next

    return sol, CGInfo(False, int(max_iter), _norm(res), r0)


def conjugate_gradient_device(
    matvec: Callable[[torch.Tensor], torch.Tensor],
    b: torch.Tensor,
    *,
    max_iter: int = 300,
    rtol: float = 1e-6,
    atol: float = 1e-6,
    check_every: int = 1,
) -> Tuple[torch.Tensor, CGInfo]:
    """``conjugate_gradient`` without preconditioner or warm start, with the vector updates,
    dot products and the stopping decision of an iteration in one device launch
    (``fs_cg_update``) instead of a dozen PyTorch launches and two host read-backs.

    The host looks at the device state every ``check_every`` iterations.  Iterations enqueued
    after the one that met the tolerance leave the iterate alone, so the solution and the
    reported iteration count are those of a loop that stopped at once; only their
    matrix-vector products are wasted, which is why large problems use ``check_every=1``.
    Same tolerance rule and ``CGInfo`` conventions as ``conjugate_gradient``.
    """
    from flash_sinkhorn_amd import _lib
    L = _lib.lib()
    rhs = b.detach().float().contiguous()
    m = rhs.numel()
    sol, res, direction = (torch.empty_like(rhs) for _ in range(3))
    state = torch.empty(8, device=rhs.device, dtype=torch.float32)
    stream = _lib.stream_of(rhs)
    _lib.check(L.fs_cg_init(rhs.data_ptr(), sol.data_ptr(), res.data_ptr(), direction.data_ptr(),
                            state.data_ptr(), m, float(rtol), float(atol), stream), "fs_cg_init")
    every = max(1, int(check_every))
    enqueued = 0
    host = None
    while enqueued < int(max_iter):
        for _ in range(min(every, int(max_iter) - enqueued)):
            a_dir = matvec(direction).float().contiguous()
            _lib.check(L.fs_cg_update(a_dir.data_ptr(), sol.data_ptr(), res.data_ptr(),
                                      direction.data_ptr(), state.data_ptr(), m, stream),
                       "fs_cg_update")
            enqueued += 1
        host = state.cpu()
        if float(host[4]) != 0.0:
            break
    if host is None:
        host = state.cpu()
    converged = float(host[5]) != 0.0
    iters = int(host[6]) if converged else int(max_iter)
    if converged:
        rnorm = float(host[3])
    else:
        rnorm = float(torch.linalg.norm(res).cpu())
    return sol, CGInfo(converged, iters, rnorm, float(host[1]))
