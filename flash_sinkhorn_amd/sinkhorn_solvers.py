"""Host loops of the two Sinkhorn solvers over the HIP log-sum-exp kernels.

Same signatures, defaults, return conventions and iteration bookkeeping as the
reference's ``sinkhorn_solvers.py`` (alternating :30-287, symmetric :290-707).
Everything device-side is one C-ABI call per step; the loops themselves are a
few lines of Python because the averaging, damping and the unbalanced shift
correction live in the kernel epilogue.
"""
from __future__ import annotations

import os
from typing import Optional, Sequence, Tuple

import torch

from flash_sinkhorn_amd import _graphs, _lib
from flash_sinkhorn_amd.kernels._common import (
    _f32c, augment_label_cost, dampening, epsilon_schedule, label_cost_active, log_weights,
    max_diameter,
)

__all__ = ["sinkhorn_flashstyle_alternating", "sinkhorn_flashstyle_symmetric"]

# Fixed-eps solves on large clouds run the kernel variant that tests a 32 x 32 logits tile after
# its hi*hi plane product (FS_FLAG_COARSE_TEST).  Each row's running maximum starts from the row's
# logit at the key that held its maximum in the step before, so on a peaked plan (small eps)
# nearly every tile ends at that test from the third step on, whatever the order of the rows.
# Whether the variant stays is decided on the device from the share of tiles that end at the
# test (FS_FLAG_COARSE_AUTO): no timing, no host read-back, the same inputs take the same path
# on every run; on a flat plan the third counted step switches to the plain kernel for good.
# None: the device decides; True / False: the coarse variant on every step / on none
COARSE_TEST = {"1": True, "0": False}.get(os.environ.get("FLASH_SINKHORN_COARSE_TEST", ""))
# measured on 8-component Gaussian mixtures at d = 8, 32, 64 and eps = 0.01: from about 20,000
# rows per cloud on the coarse variant is the faster one (25,000: 1.1-1.2x, 50,000: 1.3-1.6x,
# 100,000: 1.4-1.8x); below, its start-up per key chunk outweighs what the test saves
_COARSE_MIN_ROWS = 24000
_COARSE_MIN_STEPS = 8
# rows of 65 .. 128 columns (a kernel without carried margins, but with twice the matrix work per
# tile to save): from fewer rows on (20 alternating iterations at d = 128, eps = 0.01: 8192 rows
# per cloud 3.5 -> 3.8 ms, 12,000 rows 6.1 -> 5.1, 16,000 x 100 columns 9.3 -> 6.6, 30,000 rows
# 28.6 -> 16.1; on a flat plan, eps = 0.5 at 16,000 rows, the device's way back to the plain
# kernel costs 9.7 -> 11.1)
_COARSE_MIN_ROWS_WIDE = 10000


def _coarse_rows_ok(xf, yf):
    """Clouds large enough, and rows narrow enough, for the variant with the coarse tile test."""
    d = xf.shape[1]
    if d > 128:
        return False
    need = _COARSE_MIN_ROWS if d <= 64 else _COARSE_MIN_ROWS_WIDE
    return min(xf.shape[0], yf.shape[0]) >= need


# Reference switches from the one-launch step to two launches at this n
# (sinkhorn_solvers.py:463-468).  Both give the same numbers; here the one-launch
# step is used at every size unless the caller passes fused=False.
_FUSE_THRESHOLD = 30000


def _resolve_rho(rho, reach, rho_x, rho_y, reach_x, reach_y):
    """rho_x/rho_y beat reach_x/reach_y beat rho beats reach; reach**2 = rho."""
    if rho is not None and reach is not None:
        raise ValueError("Specify either rho or reach, not both.")
    if reach is not None:
        rho = reach ** 2
    if rho is not None:
        if rho_x is None and reach_x is None:
            rho_x = rho
        if rho_y is None and reach_y is None:
            rho_y = rho
    if reach_x is not None:
        if rho_x is not None:
            raise ValueError("Specify either rho_x or reach_x, not both.")
        rho_x = reach_x ** 2
    if reach_y is not None:
        if rho_y is not None:
            raise ValueError("Specify either rho_y or reach_y, not both.")
        rho_y = reach_y ** 2
    return rho_x, rho_y


def _require_cuda(x, y) -> None:
    # the same complaint the kernel launchers make (sinkhorn_flashstyle_sqeuclid.py:1000-1001),
    # raised before any host-side preparation touches the tensors
    if not x.is_cuda or not y.is_cuda:
        raise ValueError("x and y must be CUDA tensors")


def _max_change(f, g, prev_f, prev_g) -> float:
    return max((f - prev_f).abs().max().item(), (g - prev_g).abs().max().item())


def sinkhorn_flashstyle_alternating(
    x: torch.Tensor, y: torch.Tensor, a: torch.Tensor, b: torch.Tensor, *,
    eps: float = 0.1, n_iters: int = 100, cost_scale: float = 1.0,
    rho: Optional[float] = None, reach: Optional[float] = None,
    rho_x: Optional[float] = None, rho_y: Optional[float] = None,
    reach_x: Optional[float] = None, reach_y: Optional[float] = None,
    allow_tf32: bool = True, use_exp2: bool = True, autotune: bool = True,
    threshold: Optional[float] = None, check_every: int = 5, return_n_iters: bool = False,
    ott_convention: bool = False,
):
    """Gauss-Seidel Sinkhorn at fixed eps: f from g, then g from the NEW f.

    GeomLoss convention (default): weights inside the LSE, P = a b exp((f+g-C)/eps).
    ``ott_convention=True``: g is updated first and eps*log(weight) sits outside the
    LSE, P = exp((f+g-C)/eps).  With rho set, the kernel damps the whole shifted
    value and, as in the reference (:240-259), no shift correction follows.
    The early-stop test every ``check_every`` iterations compares against the
    potentials of the previous check (the initial ones at the first check).
    Returns (f, g) or (f, g, n_iters_used).
    """
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_lse, flashsinkhorn_lse_fused,
    )

    rho_x, rho_y = _resolve_rho(rho, reach, rho_x, rho_y, reach_x, reach_y)
    damp_f, damp_g = dampening(eps, rho_x), dampening(eps, rho_y)
    _require_cuda(x, y)
    xf, yf = x.float().contiguous(), y.float().contiguous()
    alpha = cost_scale * (xf * xf).sum(dim=1)
    beta = cost_scale * (yf * yf).sum(dim=1)
    log_a, log_b = log_weights(a), log_weights(b)
    f_hat, g_hat = -alpha, -beta
    prev_f, prev_g = (f_hat.clone(), g_hat.clone()) if threshold is not None else (None, None)
    # operand planes are converted once for the whole loop
    prepared = _lib.PreparedOperands(xf, yf, _lib.flags(use_exp2, allow_tf32))
    # the kernel variant with the coarse tile test (see COARSE_TEST): every half-update starts
    # its rows from the keys of the same half-update one iteration earlier
    coarse = False
    if (_lib.TILE_SKIP and (allow_tf32 or _lib.STRICT_OPERANDS == "fp16x2") and _coarse_rows_ok(xf, yf)
            and int(n_iters) >= _COARSE_MIN_STEPS):
        coarse = "auto" if COARSE_TEST is None else bool(COARSE_TEST)
    kw = dict(cost_scale=cost_scale, allow_tf32=allow_tf32, use_exp2=use_exp2,
              _prepared=prepared, _coarse=coarse)

    used = 0
    for it in range(int(n_iters)):
        if ott_convention:
            g_hat = eps * log_b + flashsinkhorn_lse(yf, xf, f_hat / eps, eps, damping=damp_g, **kw)
            f_hat = eps * log_a + flashsinkhorn_lse(xf, yf, g_hat / eps, eps, damping=damp_f, **kw)
        else:
            f_hat = flashsinkhorn_lse_fused(xf, yf, g_hat, log_b, eps, damping=damp_f, **kw)
            g_hat = flashsinkhorn_lse_fused(yf, xf, f_hat, log_a, eps, damping=damp_g, **kw)
        used += 1
        if threshold is not None and (it + 1) % check_every == 0:
            if _max_change(f_hat, g_hat, prev_f, prev_g) < threshold:
                break
            prev_f, prev_g = f_hat.clone(), g_hat.clone()

    f, g = f_hat + alpha, g_hat + beta
    return (f, g, used) if return_n_iters else (f, g)


def sinkhorn_flashstyle_symmetric(
    x: torch.Tensor, y: torch.Tensor, a: torch.Tensor, b: torch.Tensor, *,
    blur: float = 0.05, scaling: float = 0.5, use_epsilon_scaling: bool = True,
    last_extrapolation: bool = True, cost_scale: float = 1.0,
    eps: Optional[float] = None, n_iters: Optional[int] = None,
    diameter: Optional[float] = None, eps_list: Optional[Sequence[float]] = None,
    rho: Optional[float] = None, reach: Optional[float] = None,
    rho_x: Optional[float] = None, rho_y: Optional[float] = None,
    reach_x: Optional[float] = None, reach_y: Optional[float] = None,
    allow_tf32: bool = True, use_exp2: bool = True, autotune: bool = True,
    fused: Optional[bool] = None, threshold: Optional[float] = None, check_every: int = 5,
    return_n_iters: bool = False, return_prelast: bool = False,
    f_init: Optional[torch.Tensor] = None, g_init: Optional[torch.Tensor] = None,
    label_x: Optional[torch.Tensor] = None, label_y: Optional[torch.Tensor] = None,
    label_cost_matrix: Optional[torch.Tensor] = None, lambda_x: float = 1.0,
    lambda_y: float = 0.0, solve_info: Optional[dict] = None,
):
    """GeomLoss-style symmetric (Jacobi, averaged) Sinkhorn with an eps schedule.

    Steps: one full step at eps_list[0]; one averaged step (weight 1/2) per entry
    of eps_list; if ``last_extrapolation`` one more full step at eps_list[-1].
    Unbalanced marginals (rho_x / rho_y) enter as the per-step damping
    1/(1+eps/rho) of the soft-min, i.e. in standard potentials
    f <- (1-w) f + w*damp_f*softmin_eps(g).
    Early stop: every ``check_every`` averaged steps; the first check only takes a
    snapshot.  ``f_init``/``g_init`` warm-start (standard potentials).
    Returns (f, g[, f_prelast, g_prelast][, n_iters_used]); the prelast pair is
    only returned when ``return_prelast and last_extrapolation``.
    ``solve_info`` (not in the reference): a dict that receives ``coarse`` (the kernel variant
    of the steps: False, True or "auto") and ``prepared`` (the operand
    planes, whose ``variant_state()`` tells what the device chose).
    """
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        _symmetric_step_raw, _symmetric_steps_raw, flashsinkhorn_lse,
    )

    use_labels = label_cost_active(label_x, label_y, label_cost_matrix, lambda_y)
    if use_labels and fused is not None and not fused:
        raise ValueError("OTDD label cost requires fused=True (default). Set fused=True or omit "
                         "label_cost_matrix.")
    rho_x, rho_y = _resolve_rho(rho, reach, rho_x, rho_y, reach_x, reach_y)

    if eps_list is None:
        if use_epsilon_scaling:
            if diameter is None:
                diameter = max_diameter(x, y)
            eps_list = epsilon_schedule(diameter, blur, scaling, p=2.0)
        else:
            if eps is None or n_iters is None:
                raise ValueError("When use_epsilon_scaling=False, provide eps and n_iters")
            eps_list = [float(eps)] * int(n_iters)
    if len(eps_list) == 0:
        raise ValueError("eps_list must be non-empty")
    if n_iters is not None:
        eps_list = list(eps_list)[: int(n_iters)]

    _require_cuda(x, y)
    xf, yf = x.float().contiguous(), y.float().contiguous()
    alpha = (cost_scale * (xf * xf).sum(dim=1)).contiguous()
    beta = (cost_scale * (yf * yf).sum(dim=1)).contiguous()
    log_a, log_b = _f32c(log_weights(a)), _f32c(log_weights(b))
    f_hat = -alpha if f_init is None else _f32c(f_init) - alpha
    g_hat = -beta if g_init is None else _f32c(g_init) - beta
    if fused is None:
        fused = True
    if use_labels:
        # the label term rides in V extra feature columns; alpha / beta keep the plain norms
        xf, yf = augment_label_cost(xf, yf, label_x, label_y, label_cost_matrix, lambda_x,
                                    lambda_y)
    # Self problem OT(x, x) with one weight vector (the debiasing terms): both potentials
    # stay equal under the Jacobi iteration, so every step computes one half-update.
    if (fused and not use_labels and f_init is None and g_init is None and rho_x == rho_y
            and xf.data_ptr() == yf.data_ptr() and xf.shape == yf.shape
            and (a is b or (a.data_ptr() == b.data_ptr() and a.shape == b.shape
                            and a.stride() == b.stride()))):
        yf, beta, log_b, g_hat = xf, alpha, log_a, f_hat

    # the kernel variant with the coarse tile test (see COARSE_TEST).  On a schedule of
    # decreasing eps the plan is flat for the first steps and peaked for the last ones: the device
    # starts on the plain kernel and changes over when that kernel leaves out the exponentials
    # of most of its tiles (forcing the variant applies to fixed-eps solves only).
    coarse = False
    fixed_eps = all(e == eps_list[0] for e in eps_list)
    if (fused and not use_labels and _lib.TILE_SKIP
            and (allow_tf32 or _lib.STRICT_OPERANDS == "fp16x2") and _coarse_rows_ok(xf, yf)
            and len(eps_list) >= _COARSE_MIN_STEPS):
        if fixed_eps:
            coarse = "auto" if COARSE_TEST is None else bool(COARSE_TEST)
        elif COARSE_TEST is not False:
            coarse = "auto"
    # operand planes are converted once for the whole loop, when the first launch needs them
    # (a run replayed from a graph has planes of its own)
    made = []

    def planes():
        if not made:
            made.append(_lib.PreparedOperands(xf, yf, _lib.flags(use_exp2, allow_tf32),
                                              start_plain=(coarse == "auto" and not fixed_eps)))
        return made[0]

    def jacobi(f_hat, g_hat, e, w):
        damp_f, damp_g = dampening(e, rho_x), dampening(e, rho_y)
        if fused:
            return _symmetric_step_raw(
                xf, yf, f_hat, g_hat, log_a, log_b, e, cost_scale=cost_scale, alpha=w,
                damping_f=damp_f, damping_g=damp_g,
                shift_x=alpha if damp_f < 1.0 else None, shift_y=beta if damp_g < 1.0 else None,
                allow_tf32=allow_tf32, use_exp2=use_exp2, prepared=planes(), coarse=coarse)
        # two launches, raw-bias kernel, averaging and shift correction on the host
        kw = dict(cost_scale=cost_scale, allow_tf32=allow_tf32, use_exp2=use_exp2,
                  _prepared=planes())
        f_c = flashsinkhorn_lse(xf, yf, (g_hat + e * log_b) / e, e, damping=damp_f, **kw)
        g_c = flashsinkhorn_lse(yf, xf, (f_hat + e * log_a) / e, e, damping=damp_g, **kw)
        if damp_f < 1.0:
            f_c = f_c - alpha * (1.0 - damp_f)
        if damp_g < 1.0:
            g_c = g_c - beta * (1.0 - damp_g)
        if w == 1.0:
            return f_c, g_c
        return (1.0 - w) * f_hat + w * f_c, (1.0 - w) * g_hat + w * g_c

    def jacobi_run(f_hat, g_hat, run, with_previous=False):
        """Consecutive steps [(eps, weight), ...]: one library call when fused, replayed from a
        HIP graph on small problems (``_graphs``).  ``with_previous``: also the potentials the
        last step started from."""
        if not fused:
            f_prev, g_prev = f_hat, g_hat
            for e, w in run:
                f_prev, g_prev = f_hat, g_hat
                f_hat, g_hat = jacobi(f_hat, g_hat, e, w)
            return (f_hat, g_hat, f_prev, g_prev) if with_previous else (f_hat, g_hat)
        steps = tuple((e, w, dampening(e, rho_x), dampening(e, rho_y)) for e, w in run)
        shift_x = alpha if rho_x is not None else None
        shift_y = beta if rho_y is not None else None
        kw = dict(cost_scale=cost_scale, allow_tf32=allow_tf32, use_exp2=use_exp2,
                  with_previous=with_previous)
        if coarse is False and _graphs.eligible(xf.shape[0], yf.shape[0], len(steps), xf.device):
            aliased = yf is xf and log_b is log_a and g_hat is f_hat and beta is alpha
            flag_bits = _lib.flags(use_exp2, allow_tf32)

            def enqueue(xs, ys, fs, gs, las, lbs, sx, sy):
                if aliased:
                    ys, gs, lbs, sy = xs, fs, las, sx
                own = _lib.PreparedOperands(xs, ys, flag_bits)
                out = _symmetric_steps_raw(xs, ys, fs, gs, las, lbs, steps, shift_x=sx,
                                           shift_y=sy, prepared=own, **kw)
                return out[0::2] if aliased else out  # one vector per pair when both are one

            key = ("symmetric", xf.device.index, tuple(xf.shape), tuple(yf.shape), steps,
                   float(cost_scale), shift_x is not None, shift_y is not None, flag_bits, aliased,
                   with_previous)
            none = None
            out = _graphs.run(key, enqueue, [
                xf, none if aliased else yf, f_hat, none if aliased else g_hat, log_a,
                none if aliased else log_b, shift_x, none if aliased else shift_y])
            if aliased:
                out = tuple(t for t in out for _ in (0, 1))
            return out
        return _symmetric_steps_raw(xf, yf, f_hat, g_hat, log_a, log_b, steps, shift_x=shift_x,
                                    shift_y=shift_y, prepared=planes(), coarse=coarse, **kw)

    # the initial full step and the averaged steps, cut where a convergence check looks at
    # the potentials
    used = 0
    prev_f = prev_g = None
    f_prelast = g_prelast = None
    run = [(eps_list[0], 1.0)]
    if threshold is None and last_extrapolation:
        # nothing looks at the potentials on the way: the whole solve, extrapolation step
        # included, is one run (one library call, or one graph replay)
        run += [(e, 0.5) for e in eps_list] + [(eps_list[-1], 1.0)]
        f_hat, g_hat, f_pre, g_pre = jacobi_run(f_hat, g_hat, run, with_previous=True)
        f_prelast, g_prelast = f_pre + alpha, g_pre + beta
        used = len(run)
    else:
        for idx, e in enumerate(eps_list):
            run.append((e, 0.5))
            check = threshold is not None and (idx + 1) % check_every == 0
            if check or idx + 1 == len(eps_list):
                f_hat, g_hat = jacobi_run(f_hat, g_hat, run)
                used += len(run)
                run = []
            if check:
                if prev_f is not None and _max_change(f_hat, g_hat, prev_f, prev_g) < threshold:
                    break
                prev_f, prev_g = f_hat.clone(), g_hat.clone()
        if last_extrapolation:
            f_prelast, g_prelast = f_hat + alpha, g_hat + beta
            f_hat, g_hat = jacobi(f_hat, g_hat, eps_list[-1], 1.0)
            used += 1

    out = (f_hat + alpha, g_hat + beta)
    if return_prelast and last_extrapolation:
        out = out + (f_prelast, g_prelast)
    if solve_info is not None:
        solve_info.update(coarse=coarse, prepared=made[0] if made else None)
    if return_n_iters:
        out = out + (used,)
    return out


def sinkhorn_flashstyle_symmetric_self_pair(
    x: torch.Tensor, a: torch.Tensor, y: torch.Tensor, b: torch.Tensor, *,
    blur: float = 0.05, scaling: float = 0.5, use_epsilon_scaling: bool = True,
    last_extrapolation: bool = True, cost_scale: float = 1.0,
    eps: Optional[float] = None, n_iters: Optional[int] = None,
    rho: Optional[float] = None, allow_tf32: bool = True, use_exp2: bool = True,
    return_prelast: bool = False,
):
    """The two self problems of a debiased divergence solved together.

    Returns ``(out_x, out_y)`` where ``out_x`` is what
    ``sinkhorn_flashstyle_symmetric(x, x, a, a, ...)`` returns with the same keyword
    arguments (``rho`` standing for ``rho_x = rho_y``) and ``out_y`` likewise for
    ``(y, y, b, b)``: in a self problem both potentials stay equal, a step is one half-update,
    and the half-updates of the two problems share a launch (``fs_self_pair_steps``).  Each
    problem follows its own eps schedule (its own diameter under eps-scaling); where one
    schedule is longer, its remaining steps run alone.  No early stopping, warm start or
    label cost: callers use the single-problem solver for those.
    """
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        _self_pair_steps_raw, _symmetric_steps_raw,
    )

    def schedule(pts):
        if use_epsilon_scaling:
            lst = list(epsilon_schedule(max_diameter(pts, pts), blur, scaling, p=2.0))
        else:
            if eps is None or n_iters is None:
                raise ValueError("When use_epsilon_scaling=False, provide eps and n_iters")
            lst = [float(eps)] * int(n_iters)
        if n_iters is not None:
            lst = lst[: int(n_iters)]
        if len(lst) == 0:
            raise ValueError("eps_list must be non-empty")
        return lst

    xf, yf = x.detach().float().contiguous(), y.detach().float().contiguous()
    ex, ey = schedule(xf), schedule(yf)
    alpha_x = (cost_scale * (xf * xf).sum(dim=1)).contiguous()
    alpha_y = (cost_scale * (yf * yf).sum(dim=1)).contiguous()
    log_a, log_b = _f32c(log_weights(a.detach())), _f32c(log_weights(b.detach()))
    fx, fy = -alpha_x, -alpha_y
    shift_x = alpha_x if rho is not None else None
    shift_y = alpha_y if rho is not None else None
    flag_bits = _lib.flags(use_exp2, allow_tf32)
    kw = dict(cost_scale=cost_scale, allow_tf32=allow_tf32, use_exp2=use_exp2)
    made = []
    # the kernel variant with the coarse tile test, under the single-problem solver's conditions
    coarse = False
    fixed_eps = all(e == ex[0] for e in ex) and all(e == ey[0] for e in ey)
    if (_lib.TILE_SKIP and (allow_tf32 or _lib.STRICT_OPERANDS == "fp16x2") and _coarse_rows_ok(xf, yf)
            and min(len(ex), len(ey)) >= _COARSE_MIN_STEPS):
        if fixed_eps:
            coarse = "auto" if COARSE_TEST is None else bool(COARSE_TEST)
        elif COARSE_TEST is not False:
            coarse = "auto"  # decreasing eps: the device starts on the plain kernel

    def pair(fx, fy, steps, with_previous=False):  # steps: [(eps_x, eps_y, weight)]
        full = tuple((e1, e2, w, dampening(e1, rho), dampening(e2, rho)) for e1, e2, w in steps)
        if _graphs.eligible(max(xf.shape[0], yf.shape[0]), max(xf.shape[0], yf.shape[0]),
                            len(full), xf.device):
            def enqueue(xs, ys, fxs, fys, las, lbs, sxs, sys_):
                own = _lib.PreparedOperands(xs, ys, flag_bits, self_pair=True)
                return _self_pair_steps_raw(xs, ys, fxs, fys, las, lbs, full, shift_x=sxs,
                                            shift_y=sys_, prepared=own,
                                            with_previous=with_previous, **kw)

            key = ("self pair", xf.device.index, tuple(xf.shape), tuple(yf.shape), full,
                   float(cost_scale), shift_x is not None, flag_bits, with_previous)
            return _graphs.run(key, enqueue, [xf, yf, fx, fy, log_a, log_b, shift_x, shift_y])
        if not made:  # operand planes of both clouds, converted once for the whole loop
            made.append(_lib.PreparedOperands(xf, yf, flag_bits, self_pair=True,
                                              start_plain=(coarse == "auto" and not fixed_eps)))
        return _self_pair_steps_raw(xf, yf, fx, fy, log_a, log_b, full, shift_x=shift_x,
                                    shift_y=shift_y, prepared=made[0],
                                    with_previous=with_previous, coarse=coarse, **kw)

    def alone(pts, f, log_w, shift, steps):  # steps: [(eps, weight)]
        full = [(e, w, dampening(e, rho), dampening(e, rho)) for e, w in steps]
        return _symmetric_steps_raw(pts, pts, f, f, log_w, log_w, full, shift_x=shift,
                                    shift_y=shift, **kw)[0]

    sx = [(ex[0], 1.0)] + [(e, 0.5) for e in ex]
    sy = [(ey[0], 1.0)] + [(e, 0.5) for e in ey]
    k = min(len(sx), len(sy))
    pre_x = pre_y = None
    both = [(sx[i][0], sy[i][0], sx[i][1]) for i in range(k)]
    if len(sx) == len(sy) and last_extrapolation:
        # equal schedules: the whole solve, extrapolation step included, is one run
        fx, fy, px, py = pair(fx, fy, both + [(ex[-1], ey[-1], 1.0)], with_previous=True)
        pre_x, pre_y = px + alpha_x, py + alpha_y
    else:
        fx, fy = pair(fx, fy, both)
        if len(sx) > k:
            fx = alone(xf, fx, log_a, shift_x, sx[k:])
        if len(sy) > k:
            fy = alone(yf, fy, log_b, shift_y, sy[k:])
        if last_extrapolation:
            pre_x, pre_y = fx + alpha_x, fy + alpha_y
            fx, fy = pair(fx, fy, [(ex[-1], ey[-1], 1.0)])
    out_x = (fx + alpha_x,) * 2
    out_y = (fy + alpha_y,) * 2
    if return_prelast and last_extrapolation:
        out_x, out_y = out_x + (pre_x, pre_x), out_y + (pre_y, pre_y)
    return out_x, out_y
