"""Transport-plan products P@v, P^T@v, P@V, P^T@V on shifted potentials (HIP).

Same entry points as the reference's ``kernels/apply_flash.py``
(``apply_plan_mat_flashstyle`` :360-579, ``apply_plan_vec_flashstyle`` :835-951) with
    P_ij = a_i b_j exp((f_hat_i + g_hat_j + 2*cost_scale*x_i.y_j)/eps).
The plan is never materialised; the matrix product sweeps the keys once for all
d output columns.
"""
from __future__ import annotations

from typing import Optional

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.kernels._common import _f32c, _validate_device

__all__ = ["apply_plan_vec_flashstyle", "apply_plan_mat_flashstyle"]


def apply_plan_mat_flashstyle(
    x: torch.Tensor, y: torch.Tensor, f_hat: torch.Tensor, g_hat: torch.Tensor,
    log_a: torch.Tensor, log_b: torch.Tensor, mat: torch.Tensor, *,
    eps: float, axis: int, cost_scale: float = 1.0, scale: Optional[torch.Tensor] = None,
    block_m: Optional[int] = None, block_n: Optional[int] = None, block_k: Optional[int] = None,
    block_d: Optional[int] = None, num_warps: int = 4, num_stages: int = 2,
    use_exp2: bool = True, allow_tf32: bool = False, autotune: bool = True,
) -> torch.Tensor:
    """axis=1: P @ (mat*scale[:,None]) with mat [m,d]; axis=0: P^T @ mat with mat [n,d]."""
    if axis not in (0, 1):
        raise ValueError("axis must be 0 or 1.")
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    if x.ndim != 2 or y.ndim != 2 or mat.ndim != 2:
        raise ValueError("x, y, mat must be 2D tensors.")
    if f_hat.ndim != 1 or g_hat.ndim != 1:
        raise ValueError("f_hat and g_hat must be 1D.")
    if log_a.ndim != 1 or log_b.ndim != 1:
        raise ValueError("log_a and log_b must be 1D.")
    _validate_device(x, [("y", y), ("f_hat", f_hat), ("g_hat", g_hat), ("log_a", log_a),
                         ("log_b", log_b), ("mat", mat), ("scale", scale)])
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError("x and y must have the same feature dimension.")
    if f_hat.shape[0] != n or log_a.shape[0] != n:
        raise ValueError("f_hat and log_a must have shape (n,).")
    if g_hat.shape[0] != m or log_b.shape[0] != m:
        raise ValueError("g_hat and log_b must have shape (m,).")
    if axis == 1 and mat.shape != (m, d):
        raise ValueError("For axis=1, mat must have shape (m, d).")
    if axis == 0 and mat.shape != (n, d):
        raise ValueError("For axis=0, mat must have shape (n, d).")
    if scale is not None:
        if axis != 1:
            raise ValueError("scale is only supported for axis=1.")
        if scale.shape != (m,):
            raise ValueError("scale must have shape (m,).")
        scale = _f32c(scale)
    xf, yf, mf = _f32c(x), _f32c(y), _f32c(mat)
    fh, gh, la, lb = _f32c(f_hat), _f32c(g_hat), _f32c(log_a), _f32c(log_b)
    out = torch.empty((n if axis == 1 else m, d), device=x.device, dtype=torch.float32)
    ws = _lib.workspace(_lib.OP_APPLY_MAT, n, m, d, x.device)
    rc = _lib.lib().fs_apply_mat(
        xf.data_ptr(), yf.data_ptr(), fh.data_ptr(), gh.data_ptr(), la.data_ptr(), lb.data_ptr(),
        mf.data_ptr(), _lib.ptr(scale), out.data_ptr(), n, m, d, d, float(eps),
        2.0 * float(cost_scale), int(axis), _lib.flags(use_exp2, allow_tf32), _lib.ptr(ws),
        0 if ws is None else ws.numel(), _lib.stream_of(x))
    _lib.check(rc, "fs_apply_mat")
    return out


def apply_plan_vec_flashstyle(
    x: torch.Tensor, y: torch.Tensor, f_hat: torch.Tensor, g_hat: torch.Tensor,
    log_a: torch.Tensor, log_b: torch.Tensor, vec: torch.Tensor, *,
    eps: float, axis: int, cost_scale: float = 1.0, allow_tf32: bool = False,
    use_exp2: bool = True, block_m: int = 64, block_n: int = 64, block_k: int = 64,
    num_warps: int = 4, num_stages: int = 2,
) -> torch.Tensor:
    """axis=1: P @ vec (vec [m] -> [n]); axis=0: P^T @ vec (vec [n] -> [m])."""
    n, d = x.shape
    m = y.shape[0]
    assert f_hat.shape == (n,), f"f_hat shape {f_hat.shape} != ({n},)"
    assert g_hat.shape == (m,), f"g_hat shape {g_hat.shape} != ({m},)"
    assert log_a.shape == (n,), f"log_a shape {log_a.shape} != ({n},)"
    assert log_b.shape == (m,), f"log_b shape {log_b.shape} != ({m},)"
    if axis not in (0, 1):
        raise ValueError("axis must be 0 or 1.")
    want = m if axis == 1 else n
    assert vec.shape == (want,), f"vec shape {vec.shape} != ({want},) for axis={axis}"
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    xf, yf, vf = _f32c(x), _f32c(y), _f32c(vec)
    fh, gh, la, lb = _f32c(f_hat), _f32c(g_hat), _f32c(log_a), _f32c(log_b)
    out = torch.empty((n if axis == 1 else m,), device=x.device, dtype=torch.float32)
    ws = _lib.workspace(_lib.OP_APPLY_VEC, n, m, d, x.device)
    rc = _lib.lib().fs_apply_vec(
        xf.data_ptr(), yf.data_ptr(), fh.data_ptr(), gh.data_ptr(), la.data_ptr(), lb.data_ptr(),
        vf.data_ptr(), out.data_ptr(), n, m, d, float(eps), 2.0 * float(cost_scale), int(axis),
        _lib.flags(use_exp2, allow_tf32), _lib.ptr(ws), 0 if ws is None else ws.numel(),
        _lib.stream_of(x))
    _lib.check(rc, "fs_apply_vec")
    return out
