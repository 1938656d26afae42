"""Schur-complement matvec of the Hessian-vector path,
``out = denom * z - P^T((P z) / diag_x)``.

Mirror of the reference's ``fused_schur_matvec_sqeuclid``
(``kernels/sinkhorn_triton_apply_fused_sqeuclid.py:283-470``).  There a single kernel joins its
two plan applications with a spin-wait grid barrier and falls back to two launches when the
grid does not fit the device; here it always is two stream-ordered launches
(``fs_schur_matvec``) whose epilogues carry the element-wise factors, so the product costs two
kernel launches and their split merges and no PyTorch element-wise launch.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from flash_sinkhorn_amd import _lib
from flash_sinkhorn_amd.kernels._common import _f32c

__all__ = ["fused_schur_matvec_sqeuclid"]


def _schur_matvec_raw(x, y, f_sh, g_sh, log_a, log_b, z, inv_diag_x, denom, *, eps, cost_scale,
                      allow_tf32=False, use_exp2=True, piz=None, workspace=None):
    """Shifted potentials and log-weights as for ``apply_plan_vec_flashstyle``; every tensor
    contiguous fp32 on one device.  Returns (out [m], piz [n])."""
    n, d = x.shape
    m = y.shape[0]
    if piz is None:
        piz = torch.empty((n,), device=x.device, dtype=torch.float32)
    out = torch.empty((m,), device=x.device, dtype=torch.float32)
    ws = workspace if workspace is not None else _lib.workspace(_lib.OP_APPLY_VEC, n, m, d, x.device)
    rc = _lib.lib().fs_schur_matvec(
        x.data_ptr(), y.data_ptr(), f_sh.data_ptr(), g_sh.data_ptr(), log_a.data_ptr(),
        log_b.data_ptr(), z.data_ptr(), inv_diag_x.data_ptr(), denom.data_ptr(), piz.data_ptr(),
        out.data_ptr(), n, m, d, float(eps), 2.0 * float(cost_scale),
        _lib.flags(use_exp2, allow_tf32), _lib.ptr(ws), 0 if ws is None else ws.numel(),
        _lib.stream_of(x))
    _lib.check(rc, "fs_schur_matvec")
    return out, piz


def fused_schur_matvec_sqeuclid(
    x: torch.Tensor, y: torch.Tensor, f: torch.Tensor, g: torch.Tensor, z: torch.Tensor,
    diag_x: torch.Tensor, denom: torch.Tensor, *, eps: float,
    x2: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
    piz_buffer: Optional[torch.Tensor] = None, block_m: int = 64, block_n: int = 64,
    block_k: int = 64, num_warps: int = 4, num_stages: int = 2, use_exp2: bool = True,
    allow_tf32: bool = False, cost_scale: float = 1.0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``out = denom * z - P^T @ (P @ z / diag_x)`` with OTT-style potentials,
    ``P = exp((f + g - C) / eps)``.  Returns ``(out [m], piz_buffer [n])``; the buffer holds
    ``P @ z / diag_x`` and may be passed back in to be reused.  The tile-size arguments are
    accepted and ignored."""
    if x.ndim != 2 or y.ndim != 2:
        raise ValueError("x and y must be (n,d) and (m,d).")
    if not x.is_cuda:
        raise ValueError("CUDA required.")
    for name, t in (("y", y), ("f", f), ("g", g), ("z", z), ("diag_x", diag_x), ("denom", denom)):
        if not t.is_cuda or t.device != x.device:
            raise ValueError(f"{name} must be on the same CUDA device as x ({x.device}).")
    for name, t in (("x2", x2), ("y2", y2)):
        if t is not None and (not t.is_cuda or t.device != x.device):
            raise ValueError(f"{name} must be on the same CUDA device as x ({x.device}).")
    n, d = x.shape
    m, d2 = y.shape
    if d != d2:
        raise ValueError("x and y must have same feature dimension.")
    if f.shape[0] != n or g.shape[0] != m:
        raise ValueError("f and g shapes must match x and y.")
    if z.shape[0] != m:
        raise ValueError("z must have shape (m,).")
    if diag_x.shape[0] != n:
        raise ValueError("diag_x must have shape (n,).")
    if denom.shape[0] != m:
        raise ValueError("denom must have shape (m,).")
    xf, yf = _f32c(x), _f32c(y)
    cs, e = float(cost_scale), float(eps)
    x_sq = (xf * xf).sum(dim=1) if x2 is None else x2.float()
    y_sq = (yf * yf).sum(dim=1) if y2 is None else y2.float()
    # shifted potentials in a uniform log-weight gauge (the constants cancel inside the kernels)
    log_a = torch.full((n,), -math.log(n), device=x.device, dtype=torch.float32)
    log_b = torch.full((m,), -math.log(m), device=x.device, dtype=torch.float32)
    f_sh = (f.float() - e * log_a - cs * x_sq).contiguous()
    g_sh = (g.float() - e * log_b - cs * y_sq).contiguous()
    piz = None
    if piz_buffer is not None and piz_buffer.shape == (n,) and piz_buffer.dtype == torch.float32 \
            and piz_buffer.is_contiguous() and piz_buffer.device == x.device:
        piz = piz_buffer
    return _schur_matvec_raw(xf, yf, f_sh, g_sh, log_a, log_b, _f32c(z),
                             (1.0 / diag_x.float()).contiguous(), _f32c(denom), eps=e,
                             cost_scale=cs, allow_tf32=allow_tf32, use_exp2=use_exp2, piz=piz)
