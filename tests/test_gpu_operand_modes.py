"""The non-default operand mode of the C ABI against the fp64 oracle.

``FS_FLAG_FP32_MFMA`` (Python: ``_lib.STRICT_OPERANDS = "fp32_mfma"`` with ``allow_tf32=False``)
routes d <= 128 log-sum-exp launches to the fp32 variant of the pipelined kernel, the d <= 128
products to ``stream_kernel`` and every d > 128 operation to the column-sliced fp32-MFMA
kernels, all held to the rel 1e-4 bar of the default mode.  ``allow_tf32=True``
(``FS_FLAG_REDUCED_OPERANDS``) is a permission the library does not use: same kernels, same
numbers as the default.
"""
import numpy as np
import pytest
import torch

import oracle
from tests.golden.recipe import inputs

pytestmark = pytest.mark.gpu
RTOL = 1e-4

# d <= 128 pipelined kernel, column-sliced kernels: (wavefronts, slice) families and super-slices
SHAPES = [(300, 257, 64), (129, 1000, 3), (257, 300, 128), (100, 90, 200), (50, 140, 700),
          (600, 2000, 256), (40, 33, 1536), (40, 50, 2048)]


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def rel_err(got, want):
    got = got.detach().cpu().numpy().astype(np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def problem(n, m, d, seed=0):
    x, y, a, b = inputs(200 + seed, n, m, d, scale=1.0 / np.sqrt(max(d, 1)) * 2.0)
    rng = np.random.default_rng(seed + 11)
    f_hat = rng.standard_normal(n).astype(np.float32) * 0.3
    g_hat = rng.standard_normal(m).astype(np.float32) * 0.3
    return x, y, a, b, f_hat, g_hat


@pytest.fixture(params=["fp32_mfma"])
def strict_mode(request, monkeypatch):
    from flash_sinkhorn_amd import _lib
    monkeypatch.setattr(_lib, "STRICT_OPERANDS", request.param)
    return request.param


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_symmetric_step_in_strict_modes(strict_mode, n, m, d):
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    x, y, a, b, fh, gh = problem(n, m, d, seed=1)
    la, lb = np.log(a), np.log(b)
    wf, wg = oracle.symmetric_step(x, y, fh, gh, la, lb, 0.3, 1.0, 0.5, 1.0, 1.0)
    gf, gg = _symmetric_step_raw(*dev(x, y, fh, gh, la, lb), 0.3, cost_scale=1.0, alpha=0.5,
                                 damping_f=1.0, damping_g=1.0, allow_tf32=False)
    assert rel_err(gf, wf) < RTOL and rel_err(gg, wg) < RTOL


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_products_on_fp32_mfma(strict_mode, n, m, d):
    """With the flag every product runs on fp32 MFMA operands: `stream_kernel` for d <= 128,
    `sliced_kernel` beyond."""
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    from flash_sinkhorn_amd import c_transform_fwd
    x, y, a, b, fh, gh = problem(n, m, d, seed=2)
    la, lb = np.log(a), np.log(b)
    rng = np.random.default_rng(12)
    vm = rng.standard_normal(m).astype(np.float32)
    Vm = rng.standard_normal((m, d)).astype(np.float32)
    sc = rng.random(m).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    kw = dict(eps=0.4, cost_scale=0.5)
    got = apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, dev(vm)[0], axis=1, **kw)
    assert rel_err(got, oracle.apply_plan_vec(x, y, fh, gh, la, lb, vm, axis=1, **kw)) < RTOL
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, dev(Vm)[0], axis=1, scale=dev(sc)[0], **kw)
    assert rel_err(got, oracle.apply_plan_mat(x, y, fh, gh, la, lb, Vm, axis=1, scale=sc, **kw)) < RTOL
    wx, wy = oracle.grad_barycentric(x, y, a, b, fh, gh, 0.3, cost_scale=0.5)
    gx, gy = grad(X, Y, *dev(a, b), F, G, eps=0.3, cost_scale=0.5, allow_tf32=False)
    assert rel_err(gx, wx) < RTOL and rel_err(gy, wy) < RTOL
    A = rng.standard_normal((n, d)).astype(np.float32)
    f5 = fh - 2.0
    got = mat5_sqeuclid(*dev(x, y, f5, gh, A), eps=0.5, cost_scale=0.5)
    assert rel_err(got, oracle.mat5(x, y, f5, gh, A, 0.5, 0.5)) < RTOL
    psi = rng.standard_normal(m).astype(np.float32)
    c, idx = c_transform_fwd(X, Y, dev(psi)[0], cost_scale=0.5, allow_tf32=False)
    wc, _ = oracle.c_transform(x, y, psi, 0.5)
    scale = max(np.abs(wc).max(), 1.0)
    assert np.abs(c.cpu().numpy() - wc).max() <= 1e-5 * scale
    j = idx.cpu().numpy()
    att = 0.5 * ((x.astype(np.float64) - y.astype(np.float64)[j]) ** 2).sum(1) - psi[j]
    assert np.abs(att - wc).max() <= 2e-5 * scale


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_symmetric_step_with_allow_tf32_is_the_default_kernel(n, m, d):
    """allow_tf32=True (the reference's and this API's default) gets the same kernel as
    allow_tf32=False: bit-equal results, within 1e-4 of the oracle."""
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    x, y, a, b, fh, gh = problem(n, m, d, seed=3)
    la, lb = np.log(a), np.log(b)
    wf, wg = oracle.symmetric_step(x, y, fh, gh, la, lb, 0.3, 1.0, 0.5, 1.0, 1.0)
    args = dev(x, y, fh, gh, la, lb)
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0)
    gf, gg = _symmetric_step_raw(*args, 0.3, allow_tf32=True, **kw)
    sf, sg = _symmetric_step_raw(*args, 0.3, allow_tf32=False, **kw)
    assert rel_err(gf, wf) < RTOL and rel_err(gg, wg) < RTOL
    assert torch.equal(gf, sf) and torch.equal(gg, sg)


def test_tile_skip_leaves_results_unchanged(monkeypatch):
    """Peaked plan (small eps, clustered clouds): most 32 x 32 logits tiles lie far below the
    running row maxima and the default launch leaves their exponentials out.  The result
    must agree with the launch that computes every exponential to fp32 rounding, and with
    the oracle."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    rng = np.random.default_rng(21)
    n, m, d, eps = 3000, 4100, 64, 0.01
    cx, cy = rng.standard_normal((8, d)) * 2.0, rng.standard_normal((8, d)) * 2.0
    x = (cx[rng.integers(0, 8, n)] + rng.standard_normal((n, d))).astype(np.float32)
    y = (cy[rng.integers(0, 8, m)] + rng.standard_normal((m, d))).astype(np.float32)
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    fh = (-(x * x).sum(1)).astype(np.float32)
    gh = (-(y * y).sum(1)).astype(np.float32)
    la, lb = np.log(a), np.log(b)
    args = dev(x, y, fh, gh, la, lb)
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    monkeypatch.setattr(_lib, "TILE_SKIP", True)
    f1, g1 = _symmetric_step_raw(*args, eps, **kw)
    monkeypatch.setattr(_lib, "TILE_SKIP", False)
    f0, g0 = _symmetric_step_raw(*args, eps, **kw)
    scale = float(f0.abs().max())
    assert float((f1 - f0).abs().max()) <= 4e-7 * scale
    assert float((g1 - g0).abs().max()) <= 4e-7 * scale
    wf, wg = oracle.symmetric_step(x, y, fh, gh, la, lb, eps, 1.0, 0.5, 1.0, 1.0)
    assert rel_err(f1, wf) < RTOL and rel_err(g1, wg) < RTOL


@pytest.mark.parametrize("d", [64, 100])
def test_tile_skip_leaves_the_products_unchanged(monkeypatch, d):
    """The product kernels (gradient, plan * matrix, plan * vector) leave out the same far tiles;
    FS_FLAG_NO_TILE_SKIP (module switch TILE_SKIP = False) makes them compute every one.  On a
    peaked plan both launches must agree to fp32 rounding, with values of any magnitude."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(22)
    n, m, eps = 2100, 2600, 0.02
    sc = 0.7 / np.sqrt(d)
    centres = rng.standard_normal((8, d)) * 2.0
    x = (sc * (centres[rng.integers(0, 8, n)] + rng.standard_normal((n, d)))).astype(np.float32)
    y = (sc * (centres[rng.integers(0, 8, m)] + rng.standard_normal((m, d)))).astype(np.float32)
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    la, lb = np.log(a), np.log(b)
    fh = -(x * x).sum(1).astype(np.float32)
    gh = -(y * y).sum(1).astype(np.float32)
    for it in range(3):
        fh, gh = oracle.symmetric_step(x, y, fh, gh, la, lb, eps, 1.0, 1.0 if it == 0 else 0.5, 1.0, 1.0)
    fh, gh = fh.astype(np.float32), gh.astype(np.float32)
    f = (fh + (x * x).sum(1)).astype(np.float32)
    g = (gh + (y * y).sum(1)).astype(np.float32)
    V = (rng.standard_normal((m, d)) * 1e6).astype(np.float32)   # values far from order one
    v = (rng.standard_normal(m) * 1e6).astype(np.float32)
    X, Y, A, B, F, G, FH, GH, LA, LB, VM, VV = dev(x, y, a, b, f, g, fh, gh, la, lb, V, v)

    def run():
        gx, gy = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False)
        pm = apply_plan_mat_flashstyle(X, Y, FH, GH, LA, LB, VM, eps=eps, axis=1, allow_tf32=False)
        pv = apply_plan_vec_flashstyle(X, Y, FH, GH, LA, LB, VV, eps=eps, axis=1, allow_tf32=False)
        return gx, gy, pm, pv

    monkeypatch.setattr(_lib, "TILE_SKIP", True)
    with_skip = run()
    monkeypatch.setattr(_lib, "TILE_SKIP", False)
    without = run()
    for got, ref in zip(with_skip, without):
        assert float((got - ref).abs().max()) <= 2e-6 * float(ref.abs().max())
    wx, wy = oracle.grad_barycentric(x, y, a, b, f, g, eps)
    assert rel_err(with_skip[0], wx) < RTOL and rel_err(with_skip[1], wy) < RTOL
    want = oracle.apply_plan_mat(x, y, fh, gh, la, lb, V, eps, axis=1)
    assert rel_err(with_skip[2], want) < RTOL
    want = oracle.apply_plan_vec(x, y, fh, gh, la, lb, v, eps, axis=1)
    assert rel_err(with_skip[3], want) < RTOL
