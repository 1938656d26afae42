"""``SamplesLoss``: GeomLoss-style front end of the FlashSinkhorn path.

Same constructor arguments, call forms ``(x, y)`` / ``(a, x, b, y)``, batching,
debiasing and ``potentials=True`` behaviour as the reference's
``samples_loss.py:199-597`` (argument parsing :73-191, weight normalisation :50-70).
Squared-Euclidean cost, optionally with the OTDD label term lambda_y*W[label_i, label_j].
"""
from __future__ import annotations

import os
import warnings
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple, Union

import torch

from flash_sinkhorn_amd._autograd import _SinkhornConfig, _SinkhornCostFn
from flash_sinkhorn_amd.kernels._common import epsilon_schedule, max_diameter
from flash_sinkhorn_amd.sinkhorn_solvers import (
    sinkhorn_flashstyle_alternating, sinkhorn_flashstyle_symmetric,
    sinkhorn_flashstyle_symmetric_self_pair,
)

__all__ = ["SamplesLoss"]

# Debiased losses solve their self terms on a second stream beside the xy term (13-16 % off the
# launch-bound sizes, 2-4 % off the large ones).
DEBIAS_SIDE_STREAM = os.environ.get("FLASH_SINKHORN_DEBIAS_SIDE_STREAM", "1") != "0"
_SIDE_STREAMS: dict = {}


def _side_stream(device) -> "torch.cuda.Stream":
    key = torch.device(device).index
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
    return _SIDE_STREAMS[key]


@dataclass(frozen=True)
class _ParsedInputs:
    x: torch.Tensor
    y: torch.Tensor
    a: torch.Tensor
    b: torch.Tensor
    batched: bool
    a_view_shape: Tuple[int, ...]
    b_view_shape: Tuple[int, ...]


def _as_float_tensor(t):
    if not torch.is_tensor(t):
        raise TypeError("Expected a torch.Tensor.")
    if not t.is_floating_point():
        raise TypeError("Expected a floating-point tensor.")
    return t


def _normalize_weights(w: torch.Tensor, *, eps: float = 0.0) -> torch.Tensor:
    """w / sum(w) along the last axis (sum clamped at 1e-40)."""
    w = w.float()
    if eps > 0:
        w = w + eps
    return w / w.sum(dim=-1, keepdim=True).clamp(min=1e-40)


def _weights(w, lead: Tuple[int, ...], count: int, device, name: str, pts: str):
    """Uniform weights when absent; accept (..., count) or (..., count, 1)."""
    if w is None:
        return torch.full(lead + (count,), 1.0 / count, device=device,
                          dtype=torch.float32), lead + (count,)
    w = _as_float_tensor(w)
    if w.shape == lead + (count, 1):
        return w[..., 0], lead + (count, 1)
    if w.shape == lead + (count,):
        return w, lead + (count,)
    size = "n" if name == "a" else "m"
    if lead:
        raise ValueError(f"{name} must have shape (B,{size}) or (B,{size},1) matching {pts}.")
    raise ValueError(f"{name} must have shape ({size},) or ({size},1) matching {pts}.")


def _process_args(*args, normalize: bool) -> _ParsedInputs:
    if len(args) == 2:
        (x, y), a, b = args, None, None
    elif len(args) == 4:
        a, x, b, y = args
    else:
        raise TypeError("SamplesLoss expects either (x, y) or (a, x, b, y). "
                        f"Got {len(args)} arguments.")
    x, y = _as_float_tensor(x), _as_float_tensor(y)
    if x.ndim == 2:
        lead: Tuple[int, ...] = ()
    elif x.ndim == 3:
        if y.ndim != 3:
            raise ValueError("If x is batched (B,N,D), y must be batched too.")
        if x.shape[0] != y.shape[0]:
            raise ValueError("x and y must have the same batch size.")
        lead = (x.shape[0],)
    else:
        raise ValueError("x and y must be shaped (N,D) or (B,N,D).")
    if x.shape[-1] != y.shape[-1]:
        raise ValueError("x and y must have the same feature dimension.")
    a, a_shape = _weights(a, lead, x.shape[-2], x.device, "a", "x")
    b, b_shape = _weights(b, lead, y.shape[-2], y.device, "b", "y")
    if normalize:
        a, b = _normalize_weights(a), _normalize_weights(b)
    return _ParsedInputs(x, y, a, b, bool(lead), a_shape, b_shape)


class SamplesLoss(torch.nn.Module):
    """Entropic OT loss between weighted point clouds on one GPU.

    ``backend="symmetric"`` (default): Jacobi-averaged updates, eps-scaling,
    debiasing, balanced / unbalanced / semi-unbalanced marginals
    (``reach``, ``reach_x``, ``reach_y``; rho = reach**2).
    ``backend="alternating"``: Gauss-Seidel updates at fixed ``eps`` for ``n_iters``.
    Returns a scalar cost, a ``(B,)`` vector for batched input, or ``(f, g)`` with
    ``potentials=True`` (no autograd).  Gradients w.r.t. x, y are analytic;
    differentiating twice w.r.t. x gives the CG-based Hessian-vector product.
    """

    def __init__(
        self, loss: str = "sinkhorn", *, p: int = 2, blur: float = 0.05,
        reach: Optional[float] = None, reach_x: Optional[float] = None,
        reach_y: Optional[float] = None, scaling: float = 0.5, debias: bool = False,
        potentials: bool = False, backend: str = "symmetric", normalize: bool = True,
        use_epsilon_scaling: bool = True, last_extrapolation: bool = True,
        allow_tf32: bool = True, use_exp2: bool = True, autotune: bool = True,
        half_cost: bool = False, eps: Optional[float] = None, n_iters: Optional[int] = None,
        diameter: Optional[float] = None, eps_list: Optional[Sequence[float]] = None,
        block_m: Optional[int] = None, block_n: Optional[int] = None,
        block_k: Optional[int] = None, num_warps: Optional[int] = None, num_stages: int = 2,
        hvp_tau2: float = 1e-5, hvp_max_cg_iter: int = 300, hvp_cg_rtol: float = 1e-6,
        hvp_cg_atol: float = 1e-6, hvp_cg_stabilise_every: int = 0,
        hvp_preconditioner: str = "none", hvp_precond_terms: int = 3,
        hvp_use_preconditioner: bool = True,
        label_cost_matrix: Optional[torch.Tensor] = None, lambda_x: float = 1.0,
        lambda_y: float = 0.0, threshold: Optional[float] = None, inner_iterations: int = 10,
        use_flashstyle: Optional[bool] = None,
    ):
        super().__init__()
        if use_flashstyle is not None and not use_flashstyle:
            warnings.warn("use_flashstyle=False is deprecated. FlashSinkhorn is now the only "
                          "backend.", DeprecationWarning, stacklevel=2)
        if loss != "sinkhorn":
            raise ValueError('Only loss="sinkhorn" is supported.')
        if p != 2:
            raise ValueError("Only p=2 (squared Euclidean cost) is supported.")
        if backend not in ("symmetric", "alternating", "triton", "auto"):
            raise ValueError(
                'Only backend in {"symmetric","alternating","triton","auto"} is supported.')
        if backend in ("triton", "auto"):
            warnings.warn(f'backend="{backend}" is a legacy alias for "symmetric". '
                          'Use backend="symmetric" or backend="alternating" explicitly.',
                          DeprecationWarning, stacklevel=2)
            backend = "symmetric"
        if backend == "alternating":
            if use_epsilon_scaling:
                raise ValueError('backend="alternating" requires use_epsilon_scaling=False. '
                                 'Provide fixed eps and n_iters instead.')
            if eps is None or n_iters is None:
                raise ValueError('backend="alternating" requires eps and n_iters to be specified.')
            if label_cost_matrix is not None:
                raise ValueError('backend="alternating" does not support OTDD label cost. '
                                 'Use backend="symmetric" for label-augmented cost.')
        for nm, val, what in (("reach", reach, "balanced OT"),
                              ("reach_x", reach_x, "balanced source"),
                              ("reach_y", reach_y, "balanced target")):
            if val is not None and val <= 0:
                raise ValueError(f"{nm} must be positive (or None for {what}).")
        if reach is not None:
            reach_x = reach if reach_x is None else reach_x
            reach_y = reach if reach_y is None else reach_y

        self.loss, self.p, self.blur = loss, p, float(blur)
        self.reach_x = None if reach_x is None else float(reach_x)
        self.reach_y = None if reach_y is None else float(reach_y)
        self.rho_x = None if reach_x is None else float(reach_x) ** 2
        self.rho_y = None if reach_y is None else float(reach_y) ** 2
        same = reach_x == reach_y
        self.reach = self.reach_x if same else None
        self.rho = self.rho_x if same else None
        self.scaling, self.debias = float(scaling), bool(debias)
        self.potentials, self.backend, self.normalize = bool(potentials), backend, bool(normalize)
        self.use_epsilon_scaling = bool(use_epsilon_scaling)
        self.last_extrapolation = bool(last_extrapolation)
        self.allow_tf32, self.use_exp2, self.autotune = bool(allow_tf32), bool(use_exp2), bool(autotune)
        self.half_cost = bool(half_cost)
        self.cost_scale = 0.5 if half_cost else 1.0
        self.eps = None if eps is None else float(eps)
        self.n_iters = None if n_iters is None else int(n_iters)
        self.diameter = None if diameter is None else float(diameter)
        self.eps_list = None if eps_list is None else [float(e) for e in eps_list]
        self.block_m, self.block_n, self.block_k = block_m, block_n, block_k
        self.num_warps, self.num_stages = num_warps, int(num_stages)
        self.hvp_tau2, self.hvp_max_cg_iter = float(hvp_tau2), int(hvp_max_cg_iter)
        self.hvp_cg_rtol, self.hvp_cg_atol = float(hvp_cg_rtol), float(hvp_cg_atol)
        self.hvp_cg_stabilise_every = int(hvp_cg_stabilise_every)
        self.hvp_preconditioner = str(hvp_preconditioner)
        self.hvp_precond_terms = int(hvp_precond_terms)
        self.hvp_use_preconditioner = bool(hvp_use_preconditioner)
        self.label_cost_matrix = label_cost_matrix
        self.lambda_x, self.lambda_y = float(lambda_x), float(lambda_y)
        self.threshold = None if threshold is None else float(threshold)
        self.inner_iterations = int(inner_iterations)

    def _make_config(self) -> _SinkhornConfig:
        return _SinkhornConfig(**{k: getattr(self, k) for k in _SinkhornConfig.__dataclass_fields__})

    def _eps_list_for_inputs(self, x: torch.Tensor, y: torch.Tensor) -> Sequence[float]:
        if self.eps_list is not None:
            sched = list(self.eps_list)
        elif self.use_epsilon_scaling:
            diam = self.diameter if self.diameter is not None else max_diameter(x, y)
            sched = list(epsilon_schedule(diam, self.blur, self.scaling, p=2.0))
        else:
            if self.eps is None or self.n_iters is None:
                raise ValueError("When use_epsilon_scaling=False, provide eps and n_iters.")
            sched = [float(self.eps)] * int(self.n_iters)
        if self.n_iters is not None:
            sched = sched[: int(self.n_iters)]
        if not sched:
            raise ValueError("eps_list is empty after applying n_iters.")
        return sched

    def _solve_potentials(self, x, y, a, b, label_x, label_y):
        if self.backend == "alternating":
            sched = self._eps_list_for_inputs(x, y)
            return sinkhorn_flashstyle_alternating(
                x, y, a, b, eps=float(sched[-1]), n_iters=len(sched), cost_scale=self.cost_scale,
                reach_x=self.reach_x, reach_y=self.reach_y, allow_tf32=self.allow_tf32,
                use_exp2=self.use_exp2)
        return sinkhorn_flashstyle_symmetric(
            x, y, a, b, blur=self.blur, scaling=self.scaling,
            use_epsilon_scaling=self.use_epsilon_scaling, eps=self.eps, n_iters=self.n_iters,
            allow_tf32=self.allow_tf32, use_exp2=self.use_exp2, cost_scale=self.cost_scale,
            rho_x=self.rho_x, rho_y=self.rho_y, last_extrapolation=self.last_extrapolation,
            label_x=label_x, label_y=label_y, label_cost_matrix=self.label_cost_matrix,
            lambda_x=self.lambda_x, lambda_y=self.lambda_y, threshold=self.threshold,
            check_every=self.inner_iterations)

    def forward(self, *args: Union[torch.Tensor, float], label_x: Optional[torch.Tensor] = None,
                label_y: Optional[torch.Tensor] = None):
        parsed = _process_args(*args, normalize=self.normalize)
        if not parsed.x.is_cuda or not parsed.y.is_cuda:
            raise ValueError("flash_sinkhorn.SamplesLoss requires CUDA tensors.")
        config = self._make_config()

        def ot(xb, yb, ab, bb, lx, ly, presolved=None):
            sched = tuple(self._eps_list_for_inputs(xb, yb))
            return _SinkhornCostFn.apply(xb, yb, ab, bb, sched, config, lx, ly,
                                         self.label_cost_matrix, presolved)

        # The self terms are independent solves; without early stopping, labels or an
        # asymmetric relaxation they advance together, one launch per step for both.
        labelled = (self.label_cost_matrix is not None and label_x is not None
                    and label_y is not None and self.lambda_y != 0.0)
        pair_ok = (self.backend == "symmetric" and self.threshold is None and not labelled
                   and self.rho_x == self.rho_y)

        def solve_self_pair(xb, yb, ab, bb):
            return sinkhorn_flashstyle_symmetric_self_pair(
                xb, ab, yb, bb, blur=self.blur, scaling=self.scaling,
                use_epsilon_scaling=self.use_epsilon_scaling, eps=self.eps,
                n_iters=self.n_iters, allow_tf32=self.allow_tf32,
                use_exp2=self.use_exp2, cost_scale=self.cost_scale, rho=self.rho_x,
                last_extrapolation=self.last_extrapolation,
                return_prelast=self.last_extrapolation)

        def cost(xb, yb, ab, bb):
            # debias: OT(a,b) - OT(a,a)/2 - OT(b,b)/2
            if not (self.debias and pair_ok):
                c = ot(xb, yb, ab, bb, label_x, label_y)
                if self.debias:
                    c = c - 0.5 * ot(xb, xb, ab, ab, label_x, label_x) \
                          - 0.5 * ot(yb, yb, bb, bb, label_y, label_y)
                return c
            # The self terms run on a second stream (default priority) beside the xy solve: small
            # clouds are launch bound, and the launches of medium ones leave CUs idle.  Their
            # results are handed to this stream with an event wait, and record_stream keeps the
            # allocator from reusing them early.
            main = torch.cuda.current_stream(xb.device)
            if DEBIAS_SIDE_STREAM:
                side = _side_stream(xb.device)
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    pre_x, pre_y = solve_self_pair(xb, yb, ab, bb)
                c = ot(xb, yb, ab, bb, label_x, label_y)
                main.wait_stream(side)
                for t in pre_x + pre_y:
                    t.record_stream(main)
            else:
                pre_x, pre_y = solve_self_pair(xb, yb, ab, bb)
                c = ot(xb, yb, ab, bb, label_x, label_y)
            return c - 0.5 * ot(xb, xb, ab, ab, label_x, label_x, pre_x) \
                     - 0.5 * ot(yb, yb, bb, bb, label_y, label_y, pre_y)

        if parsed.batched:
            items = list(zip(parsed.x, parsed.y, parsed.a, parsed.b))
            if self.potentials:
                # batched potentials always use the symmetric solver
                pots = [sinkhorn_flashstyle_symmetric(
                    xb, yb, ab, bb, blur=self.blur, scaling=self.scaling,
                    use_epsilon_scaling=self.use_epsilon_scaling, eps=self.eps,
                    n_iters=self.n_iters, allow_tf32=self.allow_tf32, use_exp2=self.use_exp2,
                    cost_scale=self.cost_scale, rho_x=self.rho_x, rho_y=self.rho_y,
                    last_extrapolation=self.last_extrapolation, threshold=self.threshold,
                    check_every=self.inner_iterations) for xb, yb, ab, bb in items]
                f = torch.stack([p[0] for p in pots], dim=0).view(parsed.a_view_shape)
                g = torch.stack([p[1] for p in pots], dim=0).view(parsed.b_view_shape)
                return f, g
            return torch.stack([cost(*it) for it in items], dim=0)

        if self.potentials:
            f, g = self._solve_potentials(parsed.x, parsed.y, parsed.a, parsed.b, label_x, label_y)
            return f.view(parsed.a_view_shape), g.view(parsed.b_view_shape)
        return cost(parsed.x, parsed.y, parsed.a, parsed.b)
