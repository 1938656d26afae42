"""Seeded random sweep: every operation of the C ABI at random shapes, widths on both sides of
each kernel family's limits, against the fp64 oracle (rel 1e-4 of the largest expected value;
1e-5 for the c-transform values)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
WIDTHS = [1, 3, 7, 16, 20, 33, 64, 100, 128, 129, 160, 200, 257, 500, 777, 1030, 1536, 1600, 2050]


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def rel(got, want):
    got = got.detach().cpu().numpy().astype(np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes(seed):
    from flash_sinkhorn_amd import c_transform_fwd
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(1000 + seed)
    for _ in range(8):
        d = int(rng.choice(WIDTHS))
        n = int(rng.integers(1, 700))
        m = int(rng.integers(1, 2600 if d <= 300 else 900))
        eps = float(rng.choice([0.05, 0.3, 1.0]))
        cs = float(rng.choice([0.5, 1.0]))
        sc = float(rng.choice([0.3, 1.0, 3.0])) / np.sqrt(d)
        case = (n, m, d, eps, cs)
        x = (rng.standard_normal((n, d)) * sc).astype(np.float32)
        y = (rng.standard_normal((m, d)) * sc + 0.1 * sc).astype(np.float32)
        a = rng.dirichlet(np.ones(n)).astype(np.float32)
        b = rng.dirichlet(np.ones(m)).astype(np.float32)
        la, lb = np.log(a), np.log(b)
        f = (rng.standard_normal(n) * 0.3).astype(np.float32)   # standard potentials
        g = (rng.standard_normal(m) * 0.3).astype(np.float32)
        # shifted potentials that keep every plan entry representable in fp32
        fs = (f * eps - cs * (x.astype(np.float64) ** 2).sum(1)).astype(np.float32)
        gs = (g * eps - cs * (y.astype(np.float64) ** 2).sum(1)).astype(np.float32)
        X, Y, A, B, F, G, LA, LB, FS, GS = dev(x, y, a, b, f, g, la, lb, fs, gs)
        kw = dict(eps=eps, cost_scale=cs)

        wf, wg = oracle.symmetric_step(x, y, f, g, la, lb, eps, cs, 0.5, 0.9, 1.0)
        gf, gg = _symmetric_step_raw(X, Y, F, G, LA, LB, eps, cost_scale=cs, alpha=0.5,
                                     damping_f=0.9, damping_g=1.0, allow_tf32=False)
        assert max(rel(gf, wf), rel(gg, wg)) < 1e-4, ("step", case)

        v = rng.standard_normal(m).astype(np.float32)
        vn = rng.standard_normal(n).astype(np.float32)
        V = rng.standard_normal((m, d)).astype(np.float32)
        z = rng.random(m).astype(np.float32)
        got = apply_plan_vec_flashstyle(X, Y, FS, GS, LA, LB, dev(v)[0], axis=1, **kw)
        assert rel(got, oracle.apply_plan_vec(x, y, fs, gs, la, lb, v, axis=1, **kw)) < 1e-4, ("vec", case)
        got = apply_plan_vec_flashstyle(X, Y, FS, GS, LA, LB, dev(vn)[0], axis=0, **kw)
        assert rel(got, oracle.apply_plan_vec(x, y, fs, gs, la, lb, vn, axis=0, **kw)) < 1e-4, ("vec0", case)
        got = apply_plan_mat_flashstyle(X, Y, FS, GS, LA, LB, dev(V)[0], axis=1, scale=dev(z)[0], **kw)
        want = oracle.apply_plan_mat(x, y, fs, gs, la, lb, V, axis=1, scale=z, **kw)
        assert rel(got, want) < 1e-4, ("mat", case)

        wx, wy = oracle.grad_barycentric(x, y, a, b, f, g, eps, cost_scale=cs)
        gx, gy = grad(X, Y, A, B, F, G, eps=eps, cost_scale=cs, allow_tf32=False)
        assert max(rel(gx, wx), rel(gy, wy)) < 1e-4, ("grad", case)

        Am = rng.standard_normal((n, d)).astype(np.float32)
        f5 = f - 2.0
        got = mat5_sqeuclid(*dev(x, y, f5, g, Am), eps=eps, cost_scale=cs)
        assert rel(got, oracle.mat5(x, y, f5, g, Am, eps, cs)) < 1e-4, ("mat5", case)

        psi = rng.standard_normal(m).astype(np.float32)
        c, idx = c_transform_fwd(X, Y, dev(psi)[0], cost_scale=cs, allow_tf32=False)
        wc, _ = oracle.c_transform(x, y, psi, cs)
        scale = max(np.abs(wc).max(), 1.0)
        assert np.abs(c.cpu().numpy() - wc).max() <= 1e-5 * scale, ("c_transform", case)
        j = idx.cpu().numpy()
        att = cs * ((x.astype(np.float64) - y.astype(np.float64)[j]) ** 2).sum(1) - psi[j]
        assert np.abs(att - wc).max() <= 2e-5 * scale, ("c_transform argmin", case)
