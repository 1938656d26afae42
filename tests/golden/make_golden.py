"""Write golden vectors from the reference's own dense PyTorch implementation.

Run in the build container only (``python tests/golden/make_golden.py``): it
loads three torch-only reference files BY PATH from ``/root/reference`` (the
package ``__init__`` is never imported, so no Triton code runs), feeds them
seeded numpy inputs and stores inputs' recipe + outputs in
``tests/golden/reference_vectors.npz``.  The fixture is data only; the
reference itself never travels.

Functions pinned this way (no closed form or brute force pins their exact
iteration bookkeeping):
  * sinkhorn_geomloss_potentials_ref   (testing/reference_sinkhorn.py:119-192)
  * sinkhorn_potentials_ref            (testing/reference_sinkhorn.py:65-82)
  * sinkhorn_geomloss_*grads_ref       (testing/reference_sinkhorn.py:201-233)
  * hvp_x_dense_sqeuclid               (testing/reference_hvp.py:33-152)
  * hvp_x_dense_sqeuclid_semi_unbalanced (testing/reference_hvp.py:155-356)
"""

from __future__ import annotations

import importlib.util
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from recipe import inputs  # noqa: E402

REF = "/root/reference/src/flash_sinkhorn"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")


def _load(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def main():
    import types
    # reference_hvp.py does `from flash_sinkhorn.cg import ...`: register the
    # path-loaded cg.py under that name without importing the package.
    pkg = types.ModuleType("flash_sinkhorn")
    pkg.__path__ = []
    sys.modules["flash_sinkhorn"] = pkg
    _load("flash_sinkhorn.cg", f"{REF}/cg.py")
    rs = _load("_ref_sinkhorn", f"{REF}/testing/reference_sinkhorn.py")
    rh = _load("_ref_hvp", f"{REF}/testing/reference_hvp.py")

    T = torch.from_numpy
    out = {}

    # --- symmetric solver, fixed eps (shape of test_geomloss_sinkhorn_triton.py:42-66)
    x, y, a, b = inputs(11, 64, 48, 32)
    for tag, kw in {
        "sym_fixed": dict(use_epsilon_scaling=False, eps=0.5, n_iters=3, last_extrapolation=True),
        "sym_fixed_noext": dict(use_epsilon_scaling=False, eps=0.5, n_iters=3,
                                last_extrapolation=False),
        "sym_scaling": dict(blur=0.5, scaling=0.7, use_epsilon_scaling=True,
                            last_extrapolation=True),
        "sym_smalleps": dict(use_epsilon_scaling=False, eps=0.05, n_iters=20,
                             last_extrapolation=True),
    }.items():
        f, g = rs.sinkhorn_geomloss_potentials_ref(T(x), T(y), T(a), T(b), **kw)
        out[f"{tag}_f"] = f.numpy()
        out[f"{tag}_g"] = g.numpy()

    # --- gradients at the sym_fixed potentials
    f, g = T(out["sym_fixed_f"]), T(out["sym_fixed_g"])
    gx, gy = rs.sinkhorn_geomloss_barycentric_grads_ref(T(x), T(y), T(a), T(b), f, g, eps=0.5)
    out["grad_bary_x"], out["grad_bary_y"] = gx.numpy(), gy.numpy()
    gx, gy = rs.sinkhorn_geomloss_grads_ref(T(x), T(y), T(a), T(b), f, g, eps=0.5)
    out["grad_plan_x"], out["grad_plan_y"] = gx.numpy(), gy.numpy()

    # --- alternating solver, OTT convention (test_sinkhorn_triton.py:80-98)
    x2, y2, a2, b2 = inputs(12, 40, 56, 16)
    f, g = rs.sinkhorn_potentials_ref(T(x2), T(y2), rs.log_weights_ref(T(a2)),
                                      rs.log_weights_ref(T(b2)), eps=1.0, n_iters=5)
    out["alt_ott_f"], out["alt_ott_g"] = f.numpy(), g.numpy()

    # --- HVP (shape of test_hvp_sqeuclid.py:27-95): n=32, m=24, d=8, eps=0.2, 4 iterations
    x3, y3, a3, b3 = inputs(13, 32, 24, 8)
    rng = np.random.default_rng(113)
    A = rng.standard_normal((32, 8)).astype(np.float32)
    eps = 0.2
    fg, gg = rs.sinkhorn_geomloss_potentials_ref(
        T(x3), T(y3), T(a3), T(b3), use_epsilon_scaling=False, eps=eps, n_iters=4,
        last_extrapolation=False)
    f_ott = fg + eps * rs.log_weights_ref(T(a3))
    g_ott = gg + eps * rs.log_weights_ref(T(b3))
    out["hvp_f_ott"], out["hvp_g_ott"], out["hvp_A"] = f_ott.numpy(), g_ott.numpy(), A
    for tag, pre in (("hvp_neumann", True), ("hvp_plain", False)):
        h, info = rh.hvp_x_dense_sqeuclid(T(x3), T(y3), f_ott, g_ott, T(A), eps=eps,
                                          use_preconditioner=pre)
        out[tag] = h.numpy()
        out[f"{tag}_iters"] = np.array(info["cg_iters"])
    for tag, rx, ry in (("hvp_semi_x", 1.0, None), ("hvp_semi_y", None, 0.5),
                        ("hvp_unbal", 1.0, 2.0)):
        h, info = rh.hvp_x_dense_sqeuclid_semi_unbalanced(
            T(x3), T(y3), f_ott, g_ott, T(A), eps=eps, rho_x=rx, rho_y=ry,
            use_preconditioner=False)
        out[tag] = h.numpy()
        out[f"{tag}_iters"] = np.array(info["cg_iters"])

    np.savez_compressed(OUT, **out)
    print("wrote", OUT, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
