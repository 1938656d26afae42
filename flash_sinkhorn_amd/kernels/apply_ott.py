"""The ``Mat5`` term of the Hessian-vector product (HIP kernel).

Same entry point as the reference's ``kernels/apply_ott.py:453-566``:
    Mat5 = (-4*cost_scale/eps) * sum_j P_ij (A_i . y_j) y_j,
    P_ij = exp((f_i + g_j - cost_scale*|x_i - y_j|^2)/eps)        (OTT potentials).
The reference's deprecated OTT-convention vec/mat wrappers are not provided.
"""
from __future__ import annotations

from typing import Optional

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.kernels._common import _f32c, _validate_device

__all__ = ["mat5_sqeuclid"]


def mat5_sqeuclid(
    x: torch.Tensor, y: torch.Tensor, f: torch.Tensor, g: torch.Tensor, A: torch.Tensor, *,
    eps: float, cost_scale: float = 1.0, x2: Optional[torch.Tensor] = None,
    y2: Optional[torch.Tensor] = None, block_m: Optional[int] = None,
    block_n: Optional[int] = None, block_k: Optional[int] = None, num_warps: int = 4,
    num_stages: int = 2, use_exp2: bool = True, allow_tf32: bool = False, autotune: bool = True,
) -> torch.Tensor:
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    if x.ndim != 2 or y.ndim != 2 or A.ndim != 2:
        raise ValueError("x,y,A must be 2D tensors.")
    _validate_device(x, [("y", y), ("f", f), ("g", g), ("A", A), ("x2", x2), ("y2", y2)])
    n, d = x.shape
    m, d2 = y.shape
    if d != d2 or A.shape != (n, d):
        raise ValueError("Shapes must satisfy x:(n,d), y:(m,d), A:(n,d).")
    xf, yf, Af = _f32c(x), _f32c(y), _f32c(A)
    x2 = (xf * xf).sum(dim=1).contiguous() if x2 is None else _f32c(x2)
    y2 = (yf * yf).sum(dim=1).contiguous() if y2 is None else _f32c(y2)
    ff, gf = _f32c(f), _f32c(g)
    out = torch.empty((n, d), device=x.device, dtype=torch.float32)
    ws = _lib.workspace(_lib.OP_MAT5, n, m, d, x.device)
    rc = _lib.lib().fs_mat5(
        xf.data_ptr(), yf.data_ptr(), ff.data_ptr(), gf.data_ptr(), Af.data_ptr(), x2.data_ptr(),
        y2.data_ptr(), out.data_ptr(), n, m, d, float(eps), float(cost_scale),
        _lib.flags(use_exp2, allow_tf32), _lib.ptr(ws), 0 if ws is None else ws.numel(),
        _lib.stream_of(x))
    _lib.check(rc, "fs_mat5")
    return out
