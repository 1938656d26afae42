"""Shifted-potential log-sum-exp launchers (gfx950 HIP kernels behind a C ABI).

Same public surface as the reference's ``kernels/sinkhorn_flashstyle_sqeuclid.py``:
``flashsinkhorn_lse`` (:815-955), ``flashsinkhorn_lse_fused`` (:958-1090),
``flashsinkhorn_symmetric_step`` (:1093-1317), the precompute/bias/shift helpers
(:68-147, :1324-1363) and re-exports of the two solvers (:1370-1373).

With alpha_i = cost_scale*|x_i|^2, beta_j = cost_scale*|y_j|^2 and shifted
potentials f_hat = f - alpha, g_hat = g - beta, one half-update is
    f_hat_i = -eps * damping * LSE_j[ 2*cost_scale*x_i.y_j/eps + g_hat_j/eps + log b_j ].
Triton tuning keywords (block_*, num_warps, num_stages, autotune) are accepted
and ignored; ``use_exp2`` selects nothing (the kernels work in base 2, which is
the same function); ``allow_tf32`` selects nothing either unless
``_lib.STRICT_OPERANDS = "fp32_mfma"`` asks for fp32 MFMA operands under ``allow_tf32=False``:
the default two-plane fp16 operands are fp32-grade and the fastest mode.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.kernels._common import (_f32c, augment_label_cost, label_cost_active,
                                                log_weights)

__all__ = [
    "precompute_flashsinkhorn_inputs", "compute_bias_f", "compute_bias_g",
    "flashsinkhorn_lse", "flashsinkhorn_lse_fused", "flashsinkhorn_symmetric_step",
    "shifted_to_standard_potentials", "standard_to_shifted_potentials",
    "sinkhorn_flashstyle_alternating", "sinkhorn_flashstyle_symmetric",
]


def precompute_flashsinkhorn_inputs(x, y, a, b, eps: float, cost_scale: float = 1.0):
    """(alpha, beta, gamma, delta) = (cs|x|^2, cs|y|^2, eps*log a, eps*log b)."""
    alpha = cost_scale * (x.float() ** 2).sum(dim=1)
    beta = cost_scale * (y.float() ** 2).sum(dim=1)
    return alpha, beta, eps * log_weights(a), eps * log_weights(b)


def compute_bias_f(g, beta, delta, eps: float):
    """u = (g - beta + delta)/eps, the key bias of the f half-update."""
    return ((g - beta) + delta) / eps


def compute_bias_g(f, alpha, gamma, eps: float):
    """v = (f - alpha + gamma)/eps, the key bias of the g half-update."""
    return ((f - alpha) + gamma) / eps


def shifted_to_standard_potentials(f_hat, g_hat, alpha, beta):
    return f_hat + alpha, g_hat + beta


def standard_to_shifted_potentials(f, g, alpha, beta):
    return f - alpha, g - beta


def flashsinkhorn_lse(
    x: torch.Tensor, y: torch.Tensor, bias: torch.Tensor, eps: float, *,
    cost_scale: float = 1.0, damping: float = 1.0, allow_tf32: bool = True,
    use_exp2: bool = True, block_m: Optional[int] = None, block_n: Optional[int] = None,
    block_k: Optional[int] = None, num_warps: Optional[int] = None, num_stages: int = 2,
    autotune: bool = True, _prepared: Optional[_lib.PreparedOperands] = None, _coarse=False,
) -> torch.Tensor:
    """out_i = -eps*damping*LSE_j[2*cost_scale*x_i.y_j/eps + bias_j]; returns fp32 [n].
    ``_prepared`` / ``_coarse`` (not in the reference): operand planes converted up front, and
    the kernel variant as in ``_symmetric_step_raw``."""
    if not x.is_cuda or not y.is_cuda:
        raise ValueError("x and y must be CUDA tensors")
    if x.ndim != 2 or y.ndim != 2:
        raise ValueError("x and y must be 2D tensors")
    if bias.ndim != 1:
        raise ValueError("bias must be 1D tensor")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError("x and y must have same feature dimension")
    if bias.shape[0] != m:
        raise ValueError(f"bias must have length {m}, got {bias.shape[0]}")
    x, y, bias = _f32c(x), _f32c(y), _f32c(bias)
    out = torch.empty((n,), device=x.device, dtype=torch.float32)
    wp, wn, fl, _keep = _lib.lse_workspace(_lib.OP_LSE, x, y, _lib.flags(use_exp2, allow_tf32),
                                           _prepared)
    fl |= _lib.coarse_flag(_coarse)
    rc = _lib.lib().fs_lse(
        x.data_ptr(), y.data_ptr(), bias.data_ptr(), out.data_ptr(), n, m, d,
        float(eps), 2.0 * float(cost_scale), float(damping), fl, wp, wn, _lib.stream_of(x))
    _lib.check(rc, "fs_lse")
    return out


def flashsinkhorn_lse_fused(
    x: torch.Tensor, y: torch.Tensor, g_hat: torch.Tensor, log_w: torch.Tensor, eps: float, *,
    cost_scale: float = 1.0, damping: float = 1.0, allow_tf32: bool = True,
    use_exp2: bool = True, block_m: Optional[int] = None, block_n: Optional[int] = None,
    block_k: Optional[int] = None, num_warps: Optional[int] = None, num_stages: int = 2,
    autotune: bool = True, _prepared: Optional[_lib.PreparedOperands] = None, _coarse=False,
) -> torch.Tensor:
    """Same as flashsinkhorn_lse with bias_j = g_hat_j/eps + log_w_j formed in the kernel."""
    if not x.is_cuda or not y.is_cuda:
        raise ValueError("x and y must be CUDA tensors")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError("x and y must have same feature dimension")
    if g_hat.shape[0] != m or log_w.shape[0] != m:
        raise ValueError(f"g_hat and log_w must have length {m}")
    x, y, g_hat, log_w = _f32c(x), _f32c(y), _f32c(g_hat), _f32c(log_w)
    out = torch.empty((n,), device=x.device, dtype=torch.float32)
    wp, wn, fl, _keep = _lib.lse_workspace(_lib.OP_LSE, x, y, _lib.flags(use_exp2, allow_tf32),
                                           _prepared)
    fl |= _lib.coarse_flag(_coarse)
    rc = _lib.lib().fs_lse_fused(
        x.data_ptr(), y.data_ptr(), g_hat.data_ptr(), log_w.data_ptr(), out.data_ptr(), n, m, d,
        float(eps), 2.0 * float(cost_scale), float(damping), fl, wp, wn, _lib.stream_of(x))
    _lib.check(rc, "fs_lse_fused")
    return out


def _symmetric_step_raw(x, y, f_hat, g_hat, log_a, log_b, eps, *, cost_scale, alpha, damping_f,
                        damping_g, shift_x=None, shift_y=None, allow_tf32=True, use_exp2=True,
                        prepared=None, coarse=False):
    """One launch on already contiguous fp32 operands.  With shift_x/shift_y the
    unbalanced shift correction is applied inside the epilogue.  When every paired argument
    is the same tensor (the self problem OT(x, x)) the library computes the one distinct
    half-update and the same tensor is returned twice.  ``coarse``: True sets
    ``FS_FLAG_COARSE_TEST`` (tiles tested after their hi*hi plane product), "auto"
    ``FS_FLAG_COARSE_AUTO`` (the device decides; needs ``prepared``)."""
    n, d = x.shape
    m = y.shape[0]
    f_out = torch.empty((n,), device=x.device, dtype=torch.float32)
    self_problem = (y is x and g_hat is f_hat and log_b is log_a and shift_y is shift_x
                    and damping_f == damping_g)
    g_out = f_out if self_problem else torch.empty((m,), device=x.device, dtype=torch.float32)
    wp, wn, fl, _keep = _lib.lse_workspace(_lib.OP_SYMMETRIC_STEP, x, y,
                                           _lib.flags(use_exp2, allow_tf32), prepared)
    fl |= _lib.coarse_flag(coarse)
    rc = _lib.lib().fs_symmetric_step(
        x.data_ptr(), y.data_ptr(), f_hat.data_ptr(), g_hat.data_ptr(), log_a.data_ptr(),
        log_b.data_ptr(), f_out.data_ptr(), g_out.data_ptr(), _lib.ptr(shift_x),
        _lib.ptr(shift_y), n, m, d, float(eps), float(alpha), float(damping_f), float(damping_g),
        2.0 * float(cost_scale), fl, wp, wn, _lib.stream_of(x))
    _lib.check(rc, "fs_symmetric_step")
    return f_out, g_out


def _symmetric_steps_raw(x, y, f_hat, g_hat, log_a, log_b, steps, *, cost_scale, shift_x=None,
                         shift_y=None, allow_tf32=True, use_exp2=True, prepared=None,
                         coarse=False, with_previous=False):
    """``steps`` = [(eps, alpha, damping_f, damping_g), ...] run back to back by one library call
    (``fs_symmetric_steps``): the per-step host work is a kernel launch, not a Python round
    trip.  Operands as for ``_symmetric_step_raw``; returns the potentials of the last step,
    with ``with_previous`` followed by those the last step started from (its input: the two
    work vectors alternate, so the one before last is still intact)."""
    import ctypes
    k = len(steps)
    if k == 0:
        return (f_hat, g_hat, f_hat, g_hat) if with_previous else (f_hat, g_hat)
    n, d = x.shape
    m = y.shape[0]
    self_problem = (y is x and g_hat is f_hat and log_b is log_a and shift_y is shift_x
                    and all(s[2] == s[3] for s in steps))
    f_work = [torch.empty((n,), device=x.device, dtype=torch.float32) for _ in range(2)]
    g_work = f_work if self_problem else [
        torch.empty((m,), device=x.device, dtype=torch.float32) for _ in range(2)]
    arr = ctypes.c_float * k
    eps_a, alpha_a, df_a, dg_a = (arr(*[float(s[i]) for s in steps]) for i in range(4))
    wp, wn, fl, _keep = _lib.lse_workspace(_lib.OP_SYMMETRIC_STEP, x, y,
                                           _lib.flags(use_exp2, allow_tf32), prepared)
    fl |= _lib.coarse_flag(coarse)
    rc = _lib.lib().fs_symmetric_steps(
        x.data_ptr(), y.data_ptr(), f_hat.data_ptr(), g_hat.data_ptr(), log_a.data_ptr(),
        log_b.data_ptr(), f_work[0].data_ptr(), g_work[0].data_ptr(), f_work[1].data_ptr(),
        g_work[1].data_ptr(), _lib.ptr(shift_x), _lib.ptr(shift_y), n, m, d, eps_a, alpha_a, df_a,
        dg_a, k, 2.0 * float(cost_scale), fl, wp, wn, _lib.stream_of(x))
    _lib.check(rc, "fs_symmetric_steps")
    last = (k - 1) & 1
    f_out = f_work[last]
    out = (f_out, f_out if self_problem else g_work[last])
    if with_previous:
        f_prev = f_work[last ^ 1] if k > 1 else f_hat
        out = out + (f_prev, f_prev if self_problem else (g_work[last ^ 1] if k > 1 else g_hat))
    return out


def _self_pair_steps_raw(x, y, fx_hat, fy_hat, log_a, log_b, steps, *, cost_scale, shift_x=None,
                         shift_y=None, allow_tf32=True, use_exp2=True, prepared=None,
                         with_previous=False, coarse=False):
    """The self problems OT(x, x; a) and OT(y, y; b) advanced together (``fs_self_pair_steps``):
    ``steps`` = [(eps_x, eps_y, alpha, damping_x, damping_y), ...], one launch per step for both.
    ``prepared`` must have been built with ``self_pair=True``.  Returns (fx_hat, fy_hat), with
    ``with_previous`` followed by the pair the last step started from.  ``coarse`` as in
    ``_symmetric_step_raw``."""
    import ctypes
    k = len(steps)
    if k == 0:
        return (fx_hat, fy_hat, fx_hat, fy_hat) if with_previous else (fx_hat, fy_hat)
    n, d = x.shape
    m = y.shape[0]
    fx_work = [torch.empty((n,), device=x.device, dtype=torch.float32) for _ in range(2)]
    fy_work = [torch.empty((m,), device=x.device, dtype=torch.float32) for _ in range(2)]
    arr = ctypes.c_float * k
    ex, ey, al, dx, dy = (arr(*[float(s[i]) for s in steps]) for i in range(5))
    flag_bits = _lib.flags(use_exp2, allow_tf32)
    if prepared is not None and prepared.serves(x, y, flag_bits):
        wp, wn, fl, _keep = (prepared.ws.data_ptr(), prepared.nbytes,
                             flag_bits | _lib.FS_FLAG_OPERANDS_PREPARED, prepared.ws)
    else:
        L = _lib.lib()
        nbytes = (int(L.fs_workspace_bytes(_lib.OP_SYMMETRIC_STEP, n, n, d))
                  + int(L.fs_workspace_bytes(_lib.OP_SYMMETRIC_STEP, m, m, d)))
        _keep = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        wp, wn, fl = _keep.data_ptr(), nbytes, flag_bits
    fl |= _lib.coarse_flag(coarse)
    rc = _lib.lib().fs_self_pair_steps(
        x.data_ptr(), y.data_ptr(), fx_hat.data_ptr(), fy_hat.data_ptr(), log_a.data_ptr(),
        log_b.data_ptr(), fx_work[0].data_ptr(), fy_work[0].data_ptr(), fx_work[1].data_ptr(),
        fy_work[1].data_ptr(), _lib.ptr(shift_x), _lib.ptr(shift_y), n, m, d, ex, ey, al, dx, dy,
        k, 2.0 * float(cost_scale), fl, wp, wn, _lib.stream_of(x))
    _lib.check(rc, "fs_self_pair_steps")
    last = (k - 1) & 1
    out = (fx_work[last], fy_work[last])
    if with_previous:
        out = out + ((fx_work[last ^ 1], fy_work[last ^ 1]) if k > 1 else (fx_hat, fy_hat))
    return out


def flashsinkhorn_symmetric_step(
    x: torch.Tensor, y: torch.Tensor, f_hat: torch.Tensor, g_hat: torch.Tensor,
    log_a: torch.Tensor, log_b: torch.Tensor, eps: float, *,
    cost_scale: float = 1.0, alpha: float = 0.5, damping_f: float = 1.0, damping_g: float = 1.0,
    allow_tf32: bool = True, use_exp2: bool = True, autotune: bool = True,
    block_m: Optional[int] = None, block_n: Optional[int] = None, block_k: Optional[int] = None,
    num_warps: Optional[int] = None, num_stages: int = 2,
    label_x: Optional[torch.Tensor] = None, label_y: Optional[torch.Tensor] = None,
    label_cost_matrix: Optional[torch.Tensor] = None, lambda_x: float = 1.0,
    lambda_y: float = 0.0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Both Jacobi half-steps in one launch, each from the OLD potentials:
    f_new = (1-alpha) f_hat + alpha*(-eps*damping_f*LSE_j[...]), g_new likewise over i.
    With labels (OTDD) the dot-product term becomes lambda_x*2cs*x.y - lambda_y*cs*W[l_i, l_j],
    realised as extra feature columns (``augment_label_cost``)."""
    if not x.is_cuda or not y.is_cuda:
        raise ValueError("x and y must be CUDA tensors")
    if label_cost_active(label_x, label_y, label_cost_matrix, lambda_y):
        x, y = augment_label_cost(x, y, label_x, label_y, label_cost_matrix, lambda_x, lambda_y)
    return _symmetric_step_raw(
        _f32c(x), _f32c(y), _f32c(f_hat), _f32c(g_hat), _f32c(log_a), _f32c(log_b), eps,
        cost_scale=cost_scale, alpha=alpha, damping_f=damping_f, damping_g=damping_g,
        allow_tf32=allow_tf32, use_exp2=use_exp2)


from flash_sinkhorn_amd.sinkhorn_solvers import (  # noqa: E402
    sinkhorn_flashstyle_alternating,
    sinkhorn_flashstyle_symmetric,
)
