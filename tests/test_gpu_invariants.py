"""Invariant-style checks the reference's own test suite relies on (testing/test_half_cost.py,
test_unbalanced_sinkhorn.py:248-274 and 495-537, test_geomloss_sinkhorn_triton.py:255-322,
test_samples_loss_api.py:13-205), against the oracle where a number is involved."""
import numpy as np
import pytest
import torch

import oracle
from tests.golden.recipe import inputs

pytestmark = pytest.mark.gpu


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def rel_err(got, want):
    got = got.detach().cpu().numpy().astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def test_reach_xy_equals_reach_and_rho_is_reach_squared():
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(51, 300, 260, 16)
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(blur=0.3, allow_tf32=False)
    f1, g1 = solve(X, Y, A, B, reach=0.7, **kw)
    f2, g2 = solve(X, Y, A, B, reach_x=0.7, reach_y=0.7, **kw)
    f3, g3 = solve(X, Y, A, B, rho=0.49, **kw)
    assert torch.equal(f1, f2) and torch.equal(g1, g2)
    assert float((f1 - f3).abs().max()) < 1e-5 * float(f1.abs().max())
    fb, _ = solve(X, Y, A, B, **kw)
    assert float((f1 - fb).abs().max()) > 1e-3  # the relaxation does something


def test_half_cost_is_the_full_cost_of_rescaled_clouds():
    from flash_sinkhorn_amd import SamplesLoss
    x, y, a, b = inputs(52, 400, 350, 8)
    X, Y = dev(x, y)
    kw = dict(use_epsilon_scaling=False, eps=0.05, n_iters=30, allow_tf32=False)
    half = SamplesLoss("sinkhorn", half_cost=True, **kw)(X, Y)
    full = SamplesLoss("sinkhorn", half_cost=False, **kw)(X / 2 ** 0.5, Y / 2 ** 0.5)
    assert abs(float(half) - float(full)) < 1e-5 * abs(float(full))
    n, m = x.shape[0], y.shape[0]
    ua, ub = np.full(n, 1 / n), np.full(m, 1 / m)
    want = oracle.sinkhorn_cost(ua, ub, *oracle.sinkhorn_symmetric(
        x, y, ua, ub, use_epsilon_scaling=False, eps=0.05, n_iters=30, cost_scale=0.5), 0.05)
    assert abs(float(half) - want) < 1e-4 * abs(want)


def test_alternating_unbalanced_samples_loss_equals_direct_solver():
    from flash_sinkhorn_amd import SamplesLoss
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_alternating as solve
    x, y, a, b = inputs(53, 256, 200, 12, uniform=True)
    X, Y, A, B = dev(x, y, a, b)
    loss = SamplesLoss("sinkhorn", backend="alternating", use_epsilon_scaling=False, eps=0.1,
                       n_iters=12, reach=1.5, allow_tf32=False)(X, Y)
    f, g = solve(X, Y, A, B, eps=0.1, n_iters=12, reach=1.5, allow_tf32=False)
    wf, wg = oracle.sinkhorn_alternating(x, y, a, b, eps=0.1, n_iters=12, reach=1.5)
    assert rel_err(f, wf) < 1e-4 and rel_err(g, wg) < 1e-4
    # the alternating backend returns <a, f> + <b, g> whatever rho is (_autograd.py:339-358)
    want = float((a * wf).sum() + (b * wg).sum())
    assert abs(float(loss) - want) < 1e-4 * abs(want)


@pytest.mark.parametrize("d", [1025, 2048, 4096])
def test_large_d_gradient_matches_oracle(d):
    """The reference only sanity-checks these widths; here the dense oracle is the bar."""
    from flash_sinkhorn_amd import SamplesLoss
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(54, 48, 40, d, uniform=True, scale=1.0 / np.sqrt(d))
    X, Y, A, B = dev(x, y, a, b)
    X.requires_grad_(True)
    kw = dict(use_epsilon_scaling=False, eps=0.2, n_iters=10, allow_tf32=False)
    loss = SamplesLoss("sinkhorn", **kw)(X, Y)
    (gx,) = torch.autograd.grad(loss, X)
    assert torch.isfinite(gx).all() and float(gx.abs().max()) > 0
    _, _, fp, gp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.2,
                                             n_iters=10, return_prelast=True)
    want, _ = oracle.grad_barycentric(x, y, a, b, fp, gp, 0.2)
    assert rel_err(gx, want) < 1e-4
    f, g = solve(X.detach(), Y, A, B, **kw)
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.2, n_iters=10)
    assert rel_err(f, wf) < 1e-4 and rel_err(g, wg) < 1e-4


def test_input_forms_dtype_and_layout():
    """fp64 / fp16 inputs and non-contiguous views are cast to contiguous fp32, as the
    reference's launchers do (kernels/sinkhorn_flashstyle_sqeuclid.py:1018-1022)."""
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(55, 200, 150, 24)
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(use_epsilon_scaling=False, eps=0.3, n_iters=5, allow_tf32=False)
    f0, g0 = solve(X, Y, A, B, **kw)
    f1, g1 = solve(X.double(), Y.double(), A.double(), B.double(), **kw)
    assert f1.dtype == torch.float32 and torch.equal(f0, f1) and torch.equal(g0, g1)
    Xt = X.t().contiguous().t()  # same values, column-major storage
    assert not Xt.is_contiguous()
    f2, _ = solve(Xt, Y, A, B, **kw)
    assert torch.equal(f0, f2)
    with pytest.raises(ValueError):
        solve(X.cpu(), Y, A, B, **kw)


@pytest.mark.parametrize("lam_x,d", [(1.0, 16), (0.6, 16), (1.0, 200)])
def test_otdd_label_cost_solver_loss_and_gradient(lam_x, d):
    """Label-augmented cost (extra feature columns on the GPU) against the oracle's
    restatement of the reference formulas: potentials, debiased loss, grad_x and grad_y."""
    from flash_sinkhorn_amd import SamplesLoss
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    rng = np.random.default_rng(61)
    n, m, V = 220, 190, 5
    x, y, a, b = inputs(62, n, m, d, uniform=True, scale=1.5 / np.sqrt(d))
    lx, ly = rng.integers(0, V, n), rng.integers(0, V, m)
    W = rng.random((V, V)).astype(np.float32)
    W = (W + W.T) * 0.5
    np.fill_diagonal(W, 0.0)
    X, Y, A, B = dev(x, y, a, b)
    LX, LY, WT = torch.from_numpy(lx).cuda(), torch.from_numpy(ly).cuda(), torch.from_numpy(W).cuda()
    kw = dict(use_epsilon_scaling=False, eps=0.1, n_iters=25)
    lab = oracle.LabelCost(lx, ly, W, lam_x, 0.8)
    f, g, fp, gp = solve(X, Y, A, B, allow_tf32=False, return_prelast=True, label_x=LX,
                         label_y=LY, label_cost_matrix=WT, lambda_x=lam_x, lambda_y=0.8, **kw)
    wf, wg, wfp, wgp = oracle.sinkhorn_symmetric(x, y, a, b, return_prelast=True, label=lab, **kw)
    assert rel_err(f, wf) < 1e-4 and rel_err(g, wg) < 1e-4 and rel_err(fp, wfp) < 1e-4

    X.requires_grad_(True)
    Y.requires_grad_(True)
    L = SamplesLoss("sinkhorn", debias=True, label_cost_matrix=WT, lambda_x=lam_x, lambda_y=0.8,
                    allow_tf32=False, **kw)
    loss = L(X, Y, label_x=LX, label_y=LY)
    gx, gy = torch.autograd.grad(loss, (X, Y))

    def ot(p, q, wa, wb, lp, lq):
        lb_ = oracle.LabelCost(lp, lq, W, lam_x, 0.8)
        f_, g_, fp_, gp_ = oracle.sinkhorn_symmetric(p, q, wa, wb, return_prelast=True,
                                                     label=lb_, **kw)
        gp_x, gp_y = oracle.grad_barycentric(p, q, wa, wb, fp_, gp_, 0.1, label=lb_)
        return oracle.sinkhorn_cost(wa, wb, f_, g_, 0.1), gp_x, gp_y
    c_xy, gx_xy, gy_xy = ot(x, y, a, b, lx, ly)
    c_xx, gxx_1, gxx_2 = ot(x, x, a, a, lx, lx)
    c_yy, gyy_1, gyy_2 = ot(y, y, b, b, ly, ly)
    want = c_xy - 0.5 * c_xx - 0.5 * c_yy
    assert abs(float(loss.detach()) - want) < 1e-4 * max(abs(want), abs(c_xy) * 1e-2)
    assert rel_err(gx, gx_xy - 0.5 * (gxx_1 + gxx_2)) < 1e-4
    assert rel_err(gy, gy_xy - 0.5 * (gyy_1 + gyy_2)) < 1e-4
    with pytest.raises(NotImplementedError):
        (g1,) = torch.autograd.grad(L(X, Y, label_x=LX, label_y=LY), X, create_graph=True)
        torch.autograd.grad(g1.sum(), X)
