"""The C-ABI entry points as PyTorch custom operators (``torch.ops.flash_sinkhorn_amd.*``).

Every operator takes and returns plain tensors and Python scalars, runs the HIP library on the
current stream of its inputs' device, and carries a fake (meta) implementation that gives the
output shapes and dtypes, so the operators can be traced (``torch.compile``, ``make_fx``,
export) without a GPU.  They wrap the same launchers the rest of the package calls directly;
the package's own solver loops keep the direct calls, whose per-call host cost is lower than a
trip through the dispatcher.

=========================  =====================================================  ==================
operator                   launcher it wraps                                      C entry point
=========================  =====================================================  ==================
``lse``                    ``kernels.sinkhorn_flashstyle_sqeuclid.flashsinkhorn_lse``        ``fs_lse``
``lse_fused``              ``...flashsinkhorn_lse_fused``                          ``fs_lse_fused``
``symmetric_step``         ``...flashsinkhorn_symmetric_step``                     ``fs_symmetric_step``
``grad``                   ``kernels.sinkhorn_triton_grad_sqeuclid`` launcher      ``fs_grad``
``apply_plan_vec``         ``kernels.apply_flash.apply_plan_vec_flashstyle``       ``fs_apply_vec``
``apply_plan_mat``         ``kernels.apply_flash.apply_plan_mat_flashstyle``       ``fs_apply_mat``
``mat5``                   ``kernels.apply_ott.mat5_sqeuclid``                     ``fs_mat5``
``c_transform``            ``kernels.c_transform_sqeuclid.c_transform_kernel``     ``fs_c_transform``
``schur_matvec``           ``kernels.sinkhorn_triton_apply_fused_sqeuclid``        ``fs_schur_matvec``
=========================  =====================================================  ==================
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

__all__ = ["NAMESPACE", "OPERATORS"]

NAMESPACE = "flash_sinkhorn_amd"
OPERATORS = ("lse", "lse_fused", "symmetric_step", "grad", "apply_plan_vec", "apply_plan_mat",
             "mat5", "c_transform", "schur_matvec")


def _f32(shape, like: Tensor) -> Tensor:
    return torch.empty(shape, dtype=torch.float32, device=like.device)


@torch.library.custom_op(f"{NAMESPACE}::lse", mutates_args=())
def lse(x: Tensor, y: Tensor, bias: Tensor, eps: float, cost_scale: float = 1.0,
        damping: float = 1.0, allow_tf32: bool = False) -> Tensor:
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import flashsinkhorn_lse
    return flashsinkhorn_lse(x, y, bias, eps, cost_scale=cost_scale, damping=damping,
                             allow_tf32=allow_tf32)


@lse.register_fake
def _(x, y, bias, eps, cost_scale=1.0, damping=1.0, allow_tf32=False):
    return _f32((x.shape[0],), x)


@torch.library.custom_op(f"{NAMESPACE}::lse_fused", mutates_args=())
def lse_fused(x: Tensor, y: Tensor, pot_hat: Tensor, log_w: Tensor, eps: float,
              cost_scale: float = 1.0, damping: float = 1.0,
              allow_tf32: bool = False) -> Tensor:
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import flashsinkhorn_lse_fused
    return flashsinkhorn_lse_fused(x, y, pot_hat, log_w, eps, cost_scale=cost_scale,
                                   damping=damping, allow_tf32=allow_tf32)


@lse_fused.register_fake
def _(x, y, pot_hat, log_w, eps, cost_scale=1.0, damping=1.0, allow_tf32=False):
    return _f32((x.shape[0],), x)


@torch.library.custom_op(f"{NAMESPACE}::symmetric_step", mutates_args=())
def symmetric_step(x: Tensor, y: Tensor, f_hat: Tensor, g_hat: Tensor, log_a: Tensor,
                   log_b: Tensor, eps: float, cost_scale: float = 1.0, alpha: float = 0.5,
                   damping_f: float = 1.0, damping_g: float = 1.0,
                   allow_tf32: bool = False) -> Tuple[Tensor, Tensor]:
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_symmetric_step)
    f, g = flashsinkhorn_symmetric_step(x, y, f_hat, g_hat, log_a, log_b, eps,
                                        cost_scale=cost_scale, alpha=alpha, damping_f=damping_f,
                                        damping_g=damping_g, allow_tf32=allow_tf32)
    # the self problem with every argument aliased returns one tensor twice; operator outputs
    # may not alias
    return f, (g.clone() if g is f else g)


@symmetric_step.register_fake
def _(x, y, f_hat, g_hat, log_a, log_b, eps, cost_scale=1.0, alpha=0.5, damping_f=1.0,
      damping_g=1.0, allow_tf32=False):
    return _f32((x.shape[0],), x), _f32((y.shape[0],), x)


@torch.library.custom_op(f"{NAMESPACE}::grad", mutates_args=())
def grad(x: Tensor, y: Tensor, a: Tensor, b: Tensor, f: Tensor, g: Tensor, eps: float,
         cost_scale: float = 1.0, grad_scale: Optional[Tensor] = None,
         allow_tf32: bool = False) -> Tuple[Tensor, Tensor]:
    """Both gradients (standard potentials f, g); see ``fs_grad`` for the formula."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid)
    gx, gy = sinkhorn_geomloss_online_grad_sqeuclid(
        x, y, a, b, f, g, eps=eps, cost_scale=cost_scale, grad_scale=grad_scale,
        allow_tf32=allow_tf32)
    return gx, gy


@grad.register_fake
def _(x, y, a, b, f, g, eps, cost_scale=1.0, grad_scale=None, allow_tf32=False):
    return _f32(tuple(x.shape), x), _f32(tuple(y.shape), x)


@torch.library.custom_op(f"{NAMESPACE}::apply_plan_vec", mutates_args=())
def apply_plan_vec(x: Tensor, y: Tensor, f_hat: Tensor, g_hat: Tensor, log_a: Tensor,
                   log_b: Tensor, vec: Tensor, eps: float, axis: int, cost_scale: float = 1.0,
                   allow_tf32: bool = False) -> Tensor:
    from flash_sinkhorn_amd.kernels.apply_flash import apply_plan_vec_flashstyle
    return apply_plan_vec_flashstyle(x, y, f_hat, g_hat, log_a, log_b, vec, eps=eps, axis=axis,
                                     cost_scale=cost_scale, allow_tf32=allow_tf32)


@apply_plan_vec.register_fake
def _(x, y, f_hat, g_hat, log_a, log_b, vec, eps, axis, cost_scale=1.0, allow_tf32=False):
    return _f32((x.shape[0] if axis == 1 else y.shape[0],), x)


@torch.library.custom_op(f"{NAMESPACE}::apply_plan_mat", mutates_args=())
def apply_plan_mat(x: Tensor, y: Tensor, f_hat: Tensor, g_hat: Tensor, log_a: Tensor,
                   log_b: Tensor, mat: Tensor, eps: float, axis: int, cost_scale: float = 1.0,
                   scale: Optional[Tensor] = None, allow_tf32: bool = False) -> Tensor:
    from flash_sinkhorn_amd.kernels.apply_flash import apply_plan_mat_flashstyle
    return apply_plan_mat_flashstyle(x, y, f_hat, g_hat, log_a, log_b, mat, eps=eps, axis=axis,
                                     cost_scale=cost_scale, scale=scale, allow_tf32=allow_tf32)


@apply_plan_mat.register_fake
def _(x, y, f_hat, g_hat, log_a, log_b, mat, eps, axis, cost_scale=1.0, scale=None,
      allow_tf32=False):
    return _f32((x.shape[0] if axis == 1 else y.shape[0], mat.shape[1]), x)


@torch.library.custom_op(f"{NAMESPACE}::mat5", mutates_args=())
def mat5(x: Tensor, y: Tensor, f_ott: Tensor, g_ott: Tensor, A: Tensor, eps: float,
         cost_scale: float = 1.0, allow_tf32: bool = False) -> Tensor:
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    return mat5_sqeuclid(x, y, f_ott, g_ott, A, eps=eps, cost_scale=cost_scale,
                         allow_tf32=allow_tf32)


@mat5.register_fake
def _(x, y, f_ott, g_ott, A, eps, cost_scale=1.0, allow_tf32=False):
    return _f32(tuple(x.shape), x)


@torch.library.custom_op(f"{NAMESPACE}::c_transform", mutates_args=())
def c_transform(x: Tensor, y: Tensor, bias: Tensor, cost_scale: float = 1.0,
                allow_tf32: bool = False) -> Tuple[Tensor, Tensor]:
    from flash_sinkhorn_amd.kernels.c_transform_sqeuclid import c_transform_kernel
    return c_transform_kernel(x, y, bias, cost_scale=cost_scale, allow_tf32=allow_tf32)


@c_transform.register_fake
def _(x, y, bias, cost_scale=1.0, allow_tf32=False):
    return _f32((x.shape[0],), x), torch.empty((x.shape[0],), dtype=torch.int64, device=x.device)


@torch.library.custom_op(f"{NAMESPACE}::schur_matvec", mutates_args=())
def schur_matvec(x: Tensor, y: Tensor, f: Tensor, g: Tensor, z: Tensor, diag_x: Tensor,
                 denom: Tensor, eps: float, cost_scale: float = 1.0,
                 allow_tf32: bool = False) -> Tuple[Tensor, Tensor]:
    """(denom*z - P^T((P z)/diag_x), (P z)/diag_x) with OTT-style potentials f, g."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_fused_sqeuclid import (
        fused_schur_matvec_sqeuclid)
    return fused_schur_matvec_sqeuclid(x, y, f, g, z, diag_x, denom, eps=eps,
                                       cost_scale=cost_scale, allow_tf32=allow_tf32)


@schur_matvec.register_fake
def _(x, y, f, g, z, diag_x, denom, eps, cost_scale=1.0, allow_tf32=False):
    return _f32((y.shape[0],), x), _f32((x.shape[0],), x)
