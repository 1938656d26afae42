"""Analytic gradient of the Sinkhorn cost w.r.t. the point clouds (HIP kernel).

Same entry point as the reference's ``kernels/sinkhorn_triton_grad_sqeuclid.py:891-1207``.
The module keeps the reference's file name so existing imports keep working; there
is no Triton here.  The gradient is the softmax-weighted barycentre form
    grad_x_i = 2*cost_scale*grad_scale*a_i*(x_i - sum_j w_ij y_j),
    w_i.     = softmax_j[(g_j - C_ij)/eps + log b_j]
(and symmetrically for y), evaluated at STANDARD potentials.  Marginal relaxation
never enters this operator.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.kernels._common import (_f32c, augment_label_cost, label_cost_active,
                                                log_weights)

__all__ = ["sinkhorn_geomloss_online_grad_sqeuclid"]


def sinkhorn_geomloss_online_grad_sqeuclid(
    x: torch.Tensor, y: torch.Tensor, a: torch.Tensor, b: torch.Tensor,
    f: torch.Tensor, g: torch.Tensor, *,
    eps: float, allow_tf32: bool = True, use_exp2: bool = True,
    block_m: Optional[int] = None, block_n: Optional[int] = None,
    block_k: Optional[int] = None, num_warps: Optional[int] = None, num_stages: int = 2,
    autotune: bool = True, grad_scale: Optional[torch.Tensor] = None,
    compute_grad_x: bool = True, compute_grad_y: bool = True, cost_scale: float = 1.0,
    label_x: Optional[torch.Tensor] = None, label_y: Optional[torch.Tensor] = None,
    label_cost_matrix: Optional[torch.Tensor] = None, lambda_x: float = 1.0,
    lambda_y: float = 0.0, _seed_keys=None,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Returns (grad_x [n,d] or None, grad_y [m,d] or None), fp32.  ``grad_scale`` is a
    one-element device tensor read by the kernel (no host sync)."""
    if not x.is_cuda or not y.is_cuda:
        raise ValueError("x and y must be CUDA tensors.")
    if x.ndim != 2 or y.ndim != 2:
        raise ValueError("x and y must be 2D tensors.")
    if a.ndim != 1 or b.ndim != 1:
        raise ValueError("a and b must be 1D tensors.")
    if f.ndim != 1 or g.ndim != 1:
        raise ValueError("f and g must be 1D tensors.")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError("x and y must have the same feature dimension.")
    if a.shape[0] != n or f.shape[0] != n:
        raise ValueError("a and f shapes must match x.")
    if b.shape[0] != m or g.shape[0] != m:
        raise ValueError("b and g shapes must match y.")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise ValueError(f"Unsupported dtype for x/y: {x.dtype}")
    use_labels = label_cost_active(label_x, label_y, label_cost_matrix, lambda_y)
    compute_grad_x, compute_grad_y = bool(compute_grad_x), bool(compute_grad_y)
    if not compute_grad_x and not compute_grad_y:
        return None, None
    if grad_scale is not None:
        if grad_scale.numel() != 1:
            raise ValueError("grad_scale must be a scalar tensor.")
        if grad_scale.device != x.device:
            raise ValueError("grad_scale must be on the same device as x.")
        grad_scale = grad_scale.detach().to(dtype=torch.float32).reshape(1).contiguous()

    xf, yf = _f32c(x.detach()), _f32c(y.detach())
    x2 = (xf * xf).sum(dim=1).contiguous()
    y2 = (yf * yf).sum(dim=1).contiguous()
    x_plain, y_plain, d_plain = xf, yf, d
    if use_labels:
        # C = lambda_x*cs*|x-y|^2 + lambda_y*cs*W (reference :222-238): the weighted dot product
        # and the label term come from the augmented rows, the norms are weighted here
        xf, yf = augment_label_cost(xf, yf, label_x, label_y, label_cost_matrix, lambda_x,
                                    lambda_y)
        x2, y2 = float(lambda_x) * x2, float(lambda_x) * y2
        d = xf.shape[1]
    af, bf = _f32c(a.detach()), _f32c(b.detach())
    log_a, log_b = _f32c(log_weights(af)), _f32c(log_weights(bf))
    ff, gf = _f32c(f.detach()), _f32c(g.detach())
    gx = torch.empty((n, d), device=x.device, dtype=torch.float32) if compute_grad_x else None
    gy = torch.empty((m, d), device=x.device, dtype=torch.float32) if compute_grad_y else None
    ws = _lib.workspace(_lib.OP_GRAD, n, m, d, x.device)
    # _seed_keys: (int32 [n], int32 [m]) keys with a large logit per row, as a solve with the
    # coarse tile test leaves them (PreparedOperands.best_keys); a hint, results do not depend on it
    kx = ky = None
    if _seed_keys is not None:
        kx, ky = _seed_keys
        if (kx is None or ky is None or kx.numel() != n or ky.numel() != m
                or kx.dtype != torch.int32 or ky.dtype != torch.int32):
            kx = ky = None
    rc = _lib.lib().fs_grad_seeded(
        xf.data_ptr(), yf.data_ptr(), ff.data_ptr(), gf.data_ptr(), log_a.data_ptr(),
        log_b.data_ptr(), af.data_ptr(), bf.data_ptr(), x2.data_ptr(), y2.data_ptr(),
        _lib.ptr(grad_scale), _lib.ptr(gx), _lib.ptr(gy), n, m, d, float(eps), float(cost_scale),
        _lib.ptr(kx), _lib.ptr(ky),
        _lib.flags(use_exp2, allow_tf32), _lib.ptr(ws), 0 if ws is None else ws.numel(),
        _lib.stream_of(x))
    _lib.check(rc, "fs_grad_seeded")
    if use_labels:
        # The kernel returned 2cs*gs*w*(q' - bar(k')) on the augmented rows.  The reference's
        # result is 2*lambda_x*cs*gs*w*(q - bar(k)) on the first d columns (:277-283); with
        # x' = lambda_x*x and y' = y the two differ by a multiple of the row itself.
        lam = float(lambda_x)
        gs = 1.0 if grad_scale is None else grad_scale
        if gx is not None:
            gx = gx[:, :d_plain]
            if lam != 1.0:
                gx = lam * gx + (2.0 * cost_scale * lam * (1.0 - lam)) * gs * af[:, None] * x_plain
            gx = gx.contiguous()
        if gy is not None:
            gy = gy[:, :d_plain]
            if lam != 1.0:
                gy = gy + (2.0 * cost_scale * (lam - 1.0)) * gs * bf[:, None] * y_plain
            gy = gy.contiguous()
    return gx, gy
