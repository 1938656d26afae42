"""Cache slow fp64 ORACLE results (not reference output) so GPU tests need not recompute them.

``python tests/golden/make_oracle_fixtures.py [config1 config2 config3 config4 config5]`` writes
one ``oracle_<config>.npz`` per benchmark configuration named (all but config3 by default).  Each
takes minutes of CPU time (config3: about an hour and a half on 8 cores with
ORACLE_THREADS=8); inputs are regenerated from the seed by the ``*_inputs`` functions below,
which the tests import.  Large outputs are stored for a seeded sample of
rows only (the row indices are stored with them).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def config1_inputs():
    """n=m=2000, d=3, x,y ~ N(0,I), uniform weights (seed 1)."""
    rng = np.random.default_rng(1)
    n = 2000
    x = rng.standard_normal((n, 3)).astype(np.float32)
    y = rng.standard_normal((n, 3)).astype(np.float32)
    a = np.full(n, 1 / n, np.float32)
    return x, y, a


def config2_inputs():
    rng = np.random.default_rng(2)
    n = 10_000
    x = rng.standard_normal((n, 64)).astype(np.float32)
    y = (rng.standard_normal((n, 64)) + 0.5).astype(np.float32)
    a = np.full(n, 1 / n, np.float32)
    return x, y, a


def config4_inputs():
    """n=20000, m=30000, d=128; x ~ N(0,I), y ~ N(0,1.5^2 I); Dirichlet(1) weights with
    total masses 1.0 and 1.3 (seed 4)."""
    rng = np.random.default_rng(4)
    n, m, d = 20_000, 30_000, 128
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = (1.5 * rng.standard_normal((m, d))).astype(np.float32)
    a = rng.dirichlet(np.ones(n)).astype(np.float32)
    b = (1.3 * rng.dirichlet(np.ones(m))).astype(np.float32)
    return x, y, a, b


def config5_inputs():
    """n=m=8192, d=1536; x,y ~ N(0, I/d); uniform weights; v ~ N(0,I) (seed 5)."""
    rng = np.random.default_rng(5)
    n, d = 8192, 1536
    x = (rng.standard_normal((n, d)) / np.sqrt(d)).astype(np.float32)
    y = (rng.standard_normal((n, d)) / np.sqrt(d)).astype(np.float32)
    v = rng.standard_normal((n, d)).astype(np.float32)
    a = np.full(n, 1 / n, np.float32)
    return x, y, a, v


def _ot(x, y, a, b, eps, n_iters, cost_scale=1.0):
    """Cost from the extrapolated potentials, gradients from the pre-extrapolation ones."""
    f, g, fp, gp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps,
                                             n_iters=n_iters, cost_scale=cost_scale,
                                             return_prelast=True)
    gx, gy = oracle.grad_barycentric(x, y, a, b, fp, gp, eps, cost_scale)
    return oracle.sinkhorn_cost(a, b, f, g, eps), gx, gy, (f, g, fp, gp)


def _debiased(x, y, a, b, eps, n_iters, cost_scale=1.0):
    c, gx, _, pots = _ot(x, y, a, b, eps, n_iters, cost_scale)
    cxx, gxx_x, gxx_y, _ = _ot(x, x, a, a, eps, n_iters, cost_scale)
    cyy, _, _, _ = _ot(y, y, b, b, eps, n_iters, cost_scale)
    # x feeds both clouds of OT(x, x)
    return c - 0.5 * cxx - 0.5 * cyy, gx - 0.5 * (gxx_x + gxx_y), c, pots


def make_config1():
    x, y, a = config1_inputs()
    loss, gx, _, _ = _debiased(x, y, a, a, 0.01, 100, cost_scale=0.5)
    np.savez_compressed(os.path.join(HERE, "oracle_config1.npz"), loss=np.array(loss),
                        grad_x=gx)
    print("config1 loss", loss)


def make_config2():
    x, y, a = config2_inputs()
    loss, _, c_xy, (f, g, fp, gp) = _debiased(x, y, a, a, 0.01, 100)
    np.savez_compressed(os.path.join(HERE, "oracle_config2.npz"), f=f, g=g, f_prelast=fp,
                        g_prelast=gp, loss=np.array(c_xy), loss_debiased=np.array(loss))
    print("config2 loss", c_xy, "debiased", loss)


def config3_inputs():
    """n=m=50,000, d=64; each cloud a seeded mixture of 8 unit Gaussians with means ~ N(0, 4I);
    uniform weights (seed 3).  The generator is the benchmark's own."""
    from bench import make_inputs
    return make_inputs(50_000, 50_000, 64)


def make_config3():
    """The headline solve in fp64: 100 iterations at eps = 0.01 (102 Jacobi steps), its loss, all
    four potential vectors, and 256 sampled rows of the analytic grad_x."""
    x, y, a, b = config3_inputs()
    eps = 0.01
    f, g, fp, gp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps,
                                             n_iters=100, return_prelast=True)
    loss = oracle.sinkhorn_cost(a, b, f, g, eps)
    rows = np.sort(np.random.default_rng(33).choice(x.shape[0], 256, replace=False))
    # grad_x needs only the sampled query rows against every key
    c = oracle.sqeuclid_cost(x[rows], y)
    lg = (gp[None, :] - c) / eps + np.log(b.astype(np.float64))[None, :]
    w = np.exp(lg - lg.max(axis=1, keepdims=True))
    w /= w.sum(axis=1, keepdims=True)
    gx_rows = 2.0 * a[rows, None].astype(np.float64) * (x[rows].astype(np.float64)
                                                       - w @ y.astype(np.float64))
    np.savez_compressed(os.path.join(HERE, "oracle_config3.npz"), loss=np.array(loss), f=f, g=g,
                        f_prelast=fp, g_prelast=gp, rows=rows, grad_x_rows=gx_rows)
    print("config3 loss", loss)


def make_config4():
    x, y, a, b = config4_inputs()
    out = {}
    for tag, kw in (("reach", dict(reach=1.0)), ("semi", dict(reach_x=1.0, reach_y=None))):
        f, g, used = oracle.sinkhorn_alternating(x, y, a, b, eps=0.05 ** 2, n_iters=10,
                                                 threshold=1e-3, check_every=10,
                                                 return_n_iters=True, **kw)
        out[f"f_{tag}"], out[f"g_{tag}"], out[f"used_{tag}"] = f, g, np.array(used)
        print("config4", tag, "iterations used", used, float(np.abs(f).max()))
    np.savez_compressed(os.path.join(HERE, "oracle_config4.npz"), **out)


def make_config5():
    x, y, a, v = config5_inputs()
    eps, iters = 0.5 ** 2, 50
    loss, gx, c_xy, (f, g, fp, gp) = _debiased(x, y, a, a, eps, iters)
    rows = np.sort(np.random.default_rng(55).choice(x.shape[0], 48, replace=False))
    fo, go = oracle.geomloss_to_ott_potentials(fp, gp, a, a, eps)
    hv, info = oracle.hvp_x_from_potentials(x, y, fo, go, v, eps=eps, max_cg_iter=20)
    _, gx_xy, _, _ = _ot(x, y, a, a, eps, iters)
    np.savez_compressed(
        os.path.join(HERE, "oracle_config5.npz"), rows=rows, loss_debiased=np.array(loss),
        loss_xy=np.array(c_xy), grad_x_debiased_rows=gx[rows].astype(np.float32),
        grad_x_xy_rows=gx_xy[rows].astype(np.float32), f_prelast=fp, g_prelast=gp,
        hvp_rows=hv[rows].astype(np.float32), hvp_norm=np.array(np.linalg.norm(hv)),
        grad_x_norm=np.array(np.linalg.norm(gx)), cg_iters=np.array(info.cg_iters),
        cg_converged=np.array(info.cg_converged))
    print("config5 loss", loss, "cg iterations", info.cg_iters, info.cg_converged)


if __name__ == "__main__":
    todo = sys.argv[1:] or ["config1", "config2", "config4", "config5"]
    for name in todo:
        {"config1": make_config1, "config2": make_config2, "config3": make_config3,
         "config4": make_config4, "config5": make_config5}[name]()
