"""Oracle vs what the mathematics fixes: closed forms, brute force, invariants."""
import math

import numpy as np
import pytest
from scipy.special import logsumexp

import oracle
from tests.golden.recipe import inputs


def test_helpers_closed_forms():
    # FS/testing/test_unbalanced_sinkhorn.py:228-242 cases
    assert oracle.dampening(0.1, None) == 1.0
    assert oracle.dampening(0.1, 1.0) == pytest.approx(1.0 / 1.1, rel=1e-12)
    assert oracle.dampening(0.5, 0.25) == pytest.approx(1.0 / 3.0, rel=1e-12)
    lw = oracle.log_weights(np.array([0.5, 0.0, -1.0, 2.0]))
    assert lw.tolist() == [math.log(0.5), -100000.0, -100000.0, math.log(2.0)]
    x = np.array([[0.0, 0.0], [1.0, 2.0]]); y = np.array([[-1.0, 0.5], [3.0, 1.0]])
    assert oracle.max_diameter(x, y) == pytest.approx(math.hypot(4.0, 2.0))
    sched = oracle.epsilon_schedule(4.0, 0.5, 0.5)
    # 16, then 16,4,1 (geometric by 0.25 down to but excluding 0.25), then 0.25
    assert sched == pytest.approx([16.0, 16.0, 4.0, 1.0, 0.25])
    with pytest.raises(ValueError):
        oracle.epsilon_schedule(1.0, 0.1, 1.0)


def test_resolve_rho_priority():
    assert oracle.resolve_rho(reach=2.0) == (4.0, 4.0)
    assert oracle.resolve_rho(reach_x=3.0) == (9.0, None)
    assert oracle.resolve_rho(rho=1.0, rho_y=5.0) == (1.0, 5.0)
    with pytest.raises(ValueError):
        oracle.resolve_rho(rho=1.0, reach=1.0)
    with pytest.raises(ValueError):
        oracle.resolve_rho(rho_x=1.0, reach_x=1.0)


def test_lse_step_brute_force():
    x, y, a, b = inputs(21, 7, 5, 3)
    g = np.linspace(-1, 1, 5); eps = 0.3
    lb = np.log(b.astype(np.float64))
    want = np.empty(7)
    for i in range(7):  # python loops: nothing shared with the vectorised code
        terms = []
        for j in range(5):
            c = sum((float(x[i, k]) - float(y[j, k])) ** 2 for k in range(3))
            terms.append((g[j] - c) / eps + lb[j])
        want[i] = -eps * logsumexp(terms)
    got = oracle.softmin(x, y, g, lb, eps)
    np.testing.assert_allclose(got, want, rtol=1e-12)
    # shifted form: same thing minus |x|^2 once g is shifted by |y|^2
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    al, be = (x64 ** 2).sum(1), (y64 ** 2).sum(1)
    got_hat = oracle.lse_shifted_fused(x, y, g - be, lb, eps)
    np.testing.assert_allclose(got_hat + al, want, rtol=1e-11)
    bias = (g - be) / eps + lb
    np.testing.assert_allclose(oracle.lse_shifted(x, y, bias, eps), got_hat, rtol=1e-12)
    # bias + c  =>  out - eps*c ; damping scales the whole value
    np.testing.assert_allclose(oracle.lse_shifted(x, y, bias + 2.0, eps), got_hat - eps * 2.0,
                               rtol=1e-11)
    np.testing.assert_allclose(oracle.lse_shifted(x, y, bias, eps, damping=0.25), 0.25 * got_hat,
                               rtol=1e-12)
    # half cost halves the cross term
    got_half = oracle.lse_shifted(x, y, bias, eps, cost_scale=0.5)
    np.testing.assert_allclose(
        got_half, -eps * logsumexp((x64 @ y64.T) / eps + bias[None, :], axis=1), rtol=1e-12)


def test_symmetric_step_uses_old_potentials():
    x, y, a, b = inputs(22, 9, 6, 4)
    fh = np.linspace(-2, 0, 9); gh = np.linspace(-1, 1, 6)
    la, lb = np.log(a.astype(np.float64)), np.log(b.astype(np.float64))
    f1, g1 = oracle.symmetric_step(x, y, fh, gh, la, lb, 0.4, alpha=0.5)
    fc = oracle.lse_shifted_fused(x, y, gh, lb, 0.4)
    gc = oracle.lse_shifted_fused(y, x, fh, la, 0.4)  # OLD f, not f1
    np.testing.assert_allclose(f1, 0.5 * fh + 0.5 * fc, rtol=1e-12)
    np.testing.assert_allclose(g1, 0.5 * gh + 0.5 * gc, rtol=1e-12)


def test_balanced_fixed_point_has_right_marginals():
    x, y, a, b = inputs(23, 30, 20, 2)
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.5, n_iters=400)
    P = oracle.plan(x, y, a, b, f, g, 0.5)
    np.testing.assert_allclose(P.sum(1), a, rtol=1e-6)
    np.testing.assert_allclose(P.sum(0), b, rtol=1e-6)
    # alternating (both conventions) reaches the same plan; OTT potentials absorb eps*log w
    fa, ga = oracle.sinkhorn_alternating(x, y, a, b, eps=0.5, n_iters=400)
    np.testing.assert_allclose(oracle.plan(x, y, a, b, fa, ga, 0.5), P, rtol=1e-5, atol=1e-12)
    fo, go = oracle.sinkhorn_alternating(x, y, a, b, eps=0.5, n_iters=400, ott_convention=True)
    Po = np.exp((fo[:, None] + go[None, :] - oracle.sqeuclid_cost(x, y)) / 0.5)
    np.testing.assert_allclose(Po, P, rtol=1e-5, atol=1e-12)
    # dual cost == primal transport cost + eps*KL at the optimum
    C = oracle.sqeuclid_cost(x, y)
    ab = a.astype(np.float64)[:, None] * b.astype(np.float64)[None, :]
    primal = (P * C).sum() + 0.5 * (P * np.log(P / ab)).sum()
    assert oracle.sinkhorn_cost(a, b, f, g, 0.5) == pytest.approx(primal, rel=1e-6)


def test_unbalanced_limits_and_fixed_point():
    x, y, a, b = inputs(24, 25, 18, 3)
    kw = dict(use_epsilon_scaling=False, eps=0.3, n_iters=30)
    f0, g0 = oracle.sinkhorn_symmetric(x, y, a, b, **kw)
    f1, g1 = oracle.sinkhorn_symmetric(x, y, a, b, rho=1e12, **kw)
    np.testing.assert_allclose(f1, f0, rtol=1e-9, atol=1e-9)
    fa, ga = oracle.sinkhorn_symmetric(x, y, a, b, reach=1.5, **kw)
    fb, gb = oracle.sinkhorn_symmetric(x, y, a, b, reach_x=1.5, reach_y=1.5, **kw)
    np.testing.assert_array_equal(fa, fb)
    # unbalanced fixed point: f = damp * softmin(g)
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, rho=2.0, use_epsilon_scaling=False, eps=0.3,
                                     n_iters=500, last_extrapolation=False)
    damp = 1.0 / (1.0 + 0.3 / 2.0)
    lb = np.log(b.astype(np.float64))
    np.testing.assert_allclose(f, damp * oracle.softmin(x, y, g, lb, 0.3), rtol=1e-8)
    # alternating + rho keeps the reference's missing shift correction
    fq, gq = oracle.sinkhorn_alternating(x, y, a, b, eps=0.3, n_iters=1, rho=2.0)
    al = (x.astype(np.float64) ** 2).sum(1)
    be = (y.astype(np.float64) ** 2).sum(1)
    want = damp * oracle.softmin(x, y, np.zeros(18), lb, 0.3) + (1 - damp) * al
    np.testing.assert_allclose(fq, want, rtol=1e-10)


def _primal_kkt_residual(x, y, a, b, f, g, eps, rho_x, rho_y):
    """Stationarity of  <C,P> + eps KL(P | a b^T) + rho_x KL(P 1 | a) + rho_y KL(P^T 1 | b)  in P at
    P = a b^T exp((f + g - C)/eps), written from the primal problem (no dual update formula):
    C_ij + eps log(P_ij / a_i b_j) + rho_x log((P 1)_i / a_i) + rho_y log((P^T 1)_j / b_j) = 0;
    a balanced side (rho None) is the hard constraint P 1 = a with f_i its free multiplier."""
    a = a.astype(np.float64); b = b.astype(np.float64)
    C = np.empty((len(a), len(b)))
    for i in range(len(a)):
        for j in range(len(b)):
            C[i, j] = float(((x[i].astype(np.float64) - y[j].astype(np.float64)) ** 2).sum())
    P = a[:, None] * b[None, :] * np.exp((f[:, None] + g[None, :] - C) / eps)
    r, c = P.sum(1), P.sum(0)
    res = C + eps * np.log(P / (a[:, None] * b[None, :]))
    feas = 0.0
    if rho_x is None:
        res = res - f[:, None]
        feas = max(feas, np.abs(r / a - 1).max())
    else:
        res = res + rho_x * np.log(r / a)[:, None]
    if rho_y is None:
        res = res - g[None, :]
        feas = max(feas, np.abs(c / b - 1).max())
    else:
        res = res + rho_y * np.log(c / b)[None, :]
    return np.abs(res).max(), feas, r, c


@pytest.mark.parametrize("rho_x,rho_y", [(2.0, 0.7), (0.7, 2.0), (1.5, None), (None, 0.9)])
def test_unbalanced_symmetric_fixed_point_solves_the_primal_problem(rho_x, rho_y):
    """Pins the unbalanced / semi-unbalanced symmetric solver: at its fixed point the plan is
    stationary for the primal unbalanced problem with THESE rho_x, rho_y (a swapped rho, a
    wrong damping or a damping applied to the wrong side leaves a residual of order rho_x - rho_y),
    and the marginals obey P 1 = a exp(-f/rho_x), P^T 1 = b exp(-g/rho_y)."""
    x, y, a, b = inputs(31, 11, 9, 3)
    eps = 0.3
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, rho_x=rho_x, rho_y=rho_y,
                                     use_epsilon_scaling=False, eps=eps, n_iters=3000,
                                     last_extrapolation=False)
    res, feas, r, c = _primal_kkt_residual(x, y, a, b, f, g, eps, rho_x, rho_y)
    assert res < 1e-9 and feas < 1e-9
    if rho_x is not None:
        np.testing.assert_allclose(r, a * np.exp(-f / rho_x), rtol=1e-9)
    if rho_y is not None:
        np.testing.assert_allclose(c, b * np.exp(-g / rho_y), rtol=1e-9)
    # the check has teeth: the potentials of the problem with the two rho swapped fail it
    if rho_x != rho_y:
        fs_, gs_ = oracle.sinkhorn_symmetric(x, y, a, b, rho_x=rho_y, rho_y=rho_x,
                                             use_epsilon_scaling=False, eps=eps, n_iters=3000,
                                             last_extrapolation=False)
        bad, bad_feas, _, _ = _primal_kkt_residual(x, y, a, b, fs_, gs_, eps, rho_x, rho_y)
        assert max(bad, bad_feas) > 1e-3
    # the extrapolation step leaves a fixed point where it is
    f2, g2 = oracle.sinkhorn_symmetric(x, y, a, b, rho_x=rho_x, rho_y=rho_y,
                                       use_epsilon_scaling=False, eps=eps, n_iters=3000)
    np.testing.assert_allclose(f2, f, atol=1e-9)
    np.testing.assert_allclose(g2, g, atol=1e-9)


def test_unbalanced_symmetric_cost_is_the_primal_objective():
    """sinkhorn_cost with both marginals relaxed (FS/_autograd.py:436-455, GeomLoss's formula
    (rho+eps/2) <a, 1-exp(-f/rho)> per side) against the primal unbalanced objective evaluated
    at the fixed-point plan, through strong duality written out from the problem itself."""
    x, y, a, b = inputs(32, 10, 12, 2)
    eps, rx, ry = 0.4, 1.7, 0.6
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, rho_x=rx, rho_y=ry, use_epsilon_scaling=False,
                                     eps=eps, n_iters=3000, last_extrapolation=False)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    C = oracle.sqeuclid_cost(x, y)
    ab = a64[:, None] * b64[None, :]
    P = ab * np.exp((f[:, None] + g[None, :] - C) / eps)

    def kl(p, q):  # generalised KL between positive measures
        return float((p * np.log(p / q) - p + q).sum())

    primal = float((P * C).sum()) + eps * kl(P, ab) + rx * kl(P.sum(1), a64) + ry * kl(P.sum(0), b64)
    dual = (rx * (a64 * (1 - np.exp(-f / rx))).sum() + ry * (b64 * (1 - np.exp(-g / ry))).sum()
            - eps * (P.sum() - ab.sum()))
    assert primal == pytest.approx(dual, rel=1e-9)  # strong duality at the fixed point
    # the reference's cost formula is that dual value with eps*(m(a)m(b) - m(P)) rewritten through
    # the marginal conditions: m(P) = <a, e^{-f/rho_x}> = <b, e^{-g/rho_y}>, half to each side
    # (exact for unit masses, which `inputs` produces)
    got = oracle.sinkhorn_cost(a, b, f, g, eps, rx, ry)
    assert got == pytest.approx(dual, rel=1e-6)


def test_unbalanced_alternating_one_step_as_written_with_two_rhos():
    """The reference's alternating loop damps the whole shifted value and applies no shift
    correction (FS/sinkhorn_solvers.py:240-259; damp_f from rho_x, damp_g from rho_y, :135-136):
    f1 = damp_f softmin(g0) + (1-damp_f) |x|^2 with g0 = 0, then g1 from the NEW f1.  Written out
    with python loops for rho_x != rho_y, so that a swapped pair or a Jacobi-style g1 fails."""
    x, y, a, b = inputs(33, 6, 5, 2)
    eps, rx, ry = 0.3, 2.0, 0.5
    f1, g1 = oracle.sinkhorn_alternating(x, y, a, b, eps=eps, n_iters=1, rho_x=rx, rho_y=ry)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    df, dg = 1 / (1 + eps / rx), 1 / (1 + eps / ry)

    def smin(p, q, pot, w, i):
        t = [(pot[j] - float(((p[i] - q[j]) ** 2).sum())) / eps + math.log(w[j]) for j in range(len(q))]
        mx = max(t)
        return -eps * (mx + math.log(sum(math.exp(v - mx) for v in t)))

    want_f = np.array([df * smin(x64, y64, np.zeros(5), b, i) + (1 - df) * float((x64[i] ** 2).sum())
                       for i in range(6)])
    want_g = np.array([dg * smin(y64, x64, want_f, a, j) + (1 - dg) * float((y64[j] ** 2).sum())
                       for j in range(5)])
    np.testing.assert_allclose(f1, want_f, rtol=1e-10)
    np.testing.assert_allclose(g1, want_g, rtol=1e-10)


def test_early_stop_bookkeeping():
    x, y, a, b = inputs(25, 20, 20, 2)
    # first check only snapshots => earliest stop after 2*check_every averaged steps
    out = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=5.0, n_iters=50,
                                    threshold=1e9, check_every=3, return_n_iters=True)
    assert out[-1] == 1 + 6 + 1
    out = oracle.sinkhorn_alternating(x, y, a, b, eps=5.0, n_iters=50, threshold=1e9,
                                      check_every=3, return_n_iters=True)
    assert out[-1] == 3


def test_gradient_is_derivative_of_dual_at_fixed_potentials():
    x, y, a, b = inputs(26, 6, 5, 2)
    x = x.astype(np.float64)
    eps = 0.7
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps, n_iters=300,
                                     last_extrapolation=False)
    lb = np.log(b.astype(np.float64))

    def dual(xx):  # <a, softmin(g)> with g frozen: d/dx_i gives the barycentric gradient
        return float((a * oracle.softmin(xx, y, g, lb, eps)).sum())

    gx, _ = oracle.grad_barycentric(x, y, a, b, f, g, eps)
    fd = np.zeros_like(x)
    for i in range(6):
        for k in range(2):
            e = np.zeros_like(x); e[i, k] = 1e-6
            fd[i, k] = (dual(x + e) - dual(x - e)) / 2e-6
    np.testing.assert_allclose(gx, fd, rtol=1e-6, atol=1e-9)
    # at the balanced optimum the plan form agrees
    gp, _ = oracle.grad_plan(x, y, a, b, f, g, eps)
    np.testing.assert_allclose(gp, gx, rtol=1e-5, atol=1e-9)
    # half cost: chain rule through the sqrt(2) rescaling
    gh, _ = oracle.grad_barycentric(x, y, a, b, f, g, eps, cost_scale=0.5)
    s = math.sqrt(0.5)
    gs, _ = oracle.grad_barycentric(s * x, s * y.astype(np.float64), a, b, f, g, eps)
    np.testing.assert_allclose(gh, s * gs, rtol=1e-10)


def test_apply_and_mat5_brute_force():
    x, y, a, b = inputs(27, 5, 4, 3)
    rng = np.random.default_rng(5)
    fh, gh = rng.standard_normal(5), rng.standard_normal(4)
    la, lb = np.log(a.astype(np.float64)), np.log(b.astype(np.float64))
    v = rng.standard_normal(4); V = rng.standard_normal((4, 3)); sc = rng.random(4)
    eps, cs = 0.9, 0.5
    P = np.zeros((5, 4))
    for i in range(5):
        for j in range(4):
            dot = sum(float(x[i, k]) * float(y[j, k]) for k in range(3))
            P[i, j] = a[i] * b[j] * math.exp((fh[i] + gh[j] + 2 * cs * dot) / eps)
    kw = dict(eps=eps, cost_scale=cs)
    np.testing.assert_allclose(oracle.apply_plan_vec(x, y, fh, gh, la, lb, v, axis=1, **kw), P @ v,
                               rtol=1e-6)
    np.testing.assert_allclose(
        oracle.apply_plan_vec(x, y, fh, gh, la, lb, fh, axis=0, **kw), P.T @ fh, rtol=1e-6)
    np.testing.assert_allclose(
        oracle.apply_plan_mat(x, y, fh, gh, la, lb, V, axis=1, scale=sc, **kw),
        P @ (V * sc[:, None]), rtol=1e-6)
    W = rng.standard_normal((5, 3))
    np.testing.assert_allclose(oracle.apply_plan_mat(x, y, fh, gh, la, lb, W, axis=0, **kw),
                               P.T @ W, rtol=1e-6)
    with pytest.raises(ValueError):
        oracle.apply_plan_mat(x, y, fh, gh, la, lb, W, axis=0, scale=sc, **kw)
    # mat5 with OTT potentials
    A = rng.standard_normal((5, 3))
    fo, go = rng.standard_normal(5), rng.standard_normal(4)
    want = np.zeros((5, 3))
    for i in range(5):
        for j in range(4):
            c = cs * sum((float(x[i, k]) - float(y[j, k])) ** 2 for k in range(3))
            p = math.exp((fo[i] + go[j] - c) / eps)
            ay = sum(A[i, k] * float(y[j, k]) for k in range(3))
            want[i] += p * ay * y[j]
    np.testing.assert_allclose(oracle.mat5(x, y, fo, go, A, eps, cs), (-4 * cs / eps) * want,
                               rtol=1e-6)


def test_cg_matches_dense_solve_and_bookkeeping():
    rng = np.random.default_rng(3)
    M = rng.standard_normal((12, 12)); M = M @ M.T + 12 * np.eye(12)
    b = rng.standard_normal(12)
    x, info = oracle.conjugate_gradient(lambda v: M @ v, b, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(x, np.linalg.solve(M, b), rtol=1e-9)
    assert info.cg_converged and info.cg_iters <= 12
    _, info = oracle.conjugate_gradient(lambda v: M @ v, b, max_iter=2, rtol=1e-14, atol=0.0)
    assert (not info.cg_converged) and info.cg_iters == 2
    x, info = oracle.conjugate_gradient(lambda v: M @ v, b, x0=np.linalg.solve(M, b))
    assert info.cg_iters == 1 or info.cg_initial_residual < 1e-10
    d = np.diag(M)
    x, _ = oracle.conjugate_gradient(lambda v: M @ v, b, preconditioner=lambda r: r / d,
                                     rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(x, np.linalg.solve(M, b), rtol=1e-9)


def test_hvp_matches_finite_difference_of_gradient():
    # Full cost, balanced: d/dt grad_x OT(x + tA, y) at a converged solve equals the HVP (up
    # to the tau2 regularisation).  A dropped Mat term or wrong sign fails this.
    x, y, a, b = inputs(28, 10, 8, 2)
    x = x.astype(np.float64); y = y.astype(np.float64)
    rng = np.random.default_rng(9)
    A = rng.standard_normal(x.shape)
    eps = 0.8

    def grad(xx):
        f, g = oracle.sinkhorn_symmetric(xx, y, a, b, use_epsilon_scaling=False, eps=eps,
                                         n_iters=3000, last_extrapolation=False)
        return oracle.grad_barycentric(xx, y, a, b, f, g, eps)[0]

    f, g = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps, n_iters=3000,
                                     last_extrapolation=False)
    fo, go = oracle.geomloss_to_ott_potentials(f, g, a, b, eps)
    h, info = oracle.hvp_x_from_potentials(x, y, fo, go, A, eps=eps, tau2=1e-9, cg_rtol=1e-12,
                                           cg_atol=1e-14)
    t = 1e-5
    fd = (grad(x + t * A) - grad(x - t * A)) / (2 * t)
    np.testing.assert_allclose(h, fd, rtol=2e-4, atol=1e-7)


def test_label_cost_formulas_brute_force():
    """LabelCost restates two reference formulas; check both against python loops and the
    solver against a dense iteration written out independently."""
    rng = np.random.default_rng(21)
    n, m, d, V = 7, 6, 3, 4
    x, y = rng.standard_normal((n, d)), rng.standard_normal((m, d))
    lx, ly = rng.integers(0, V, n), rng.integers(0, V, m)
    W = rng.random((V, V)) * 2.0
    lab = oracle.LabelCost(lx, ly, W, lambda_x=0.7, lambda_y=1.3)
    cs = 0.5
    step = lab.step_cost(x, y, 0, n, cs, np.float64)
    grad = lab.grad_cost(x, y, cs, np.float64)
    for i in range(n):
        for j in range(m):
            dot = float(x[i] @ y[j])
            want_step = cs * (x[i] @ x[i] + y[j] @ y[j]) - 0.7 * 2 * cs * dot + 1.3 * cs * W[lx[i], ly[j]]
            want_grad = 0.7 * cs * float(((x[i] - y[j]) ** 2).sum()) + 1.3 * cs * W[lx[i], ly[j]]
            assert abs(step[i, j] - want_step) < 1e-12 and abs(grad[i, j] - want_grad) < 1e-12
    np.testing.assert_allclose(lab.swapped().step_cost(y, x, 0, m, cs, np.float64), step.T, atol=1e-12)
    # solver: with lambda_x = 1 the label problem is the plain problem on cost C + lambda_y*cs*W
    a, b = np.full(n, 1 / n), np.full(m, 1 / m)
    lab1 = oracle.LabelCost(lx, ly, W, 1.0, 1.3)
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.3, n_iters=200,
                                     cost_scale=cs, label=lab1)
    C = lab1.grad_cost(x, y, cs, np.float64)
    P = a[:, None] * b[None, :] * np.exp((f[:, None] + g[None, :] - C) / 0.3)
    np.testing.assert_allclose(P.sum(1), a, rtol=1e-6)
    np.testing.assert_allclose(P.sum(0), b, rtol=1e-6)
    gx, gy = oracle.grad_barycentric(x, y, a, b, f, g, 0.3, cs, label=lab1)
    np.testing.assert_allclose(gx, 2 * cs * (a[:, None] * x - P @ y), rtol=1e-5, atol=1e-9)


def test_implicit_gradient_matches_finite_differences():
    """The implicit-function-theorem gradient (full cost) is the derivative of
    <gf, f*(x)> + <gg, g*(x)> through the converged potentials, for a loss that does not see
    the (c, -c) gauge of the potentials."""
    rng = np.random.default_rng(0)
    n, m, d, eps = 6, 5, 2, 0.5
    x, y = rng.standard_normal((n, d)), rng.standard_normal((m, d))
    a = rng.random(n) + 0.5; a /= a.sum()
    b = rng.random(m) + 0.5; b /= b.sum()
    gf, gg = rng.standard_normal(n), rng.standard_normal(m)
    gg += (gf.sum() - gg.sum()) / m

    def potentials(xx):
        return oracle.sinkhorn_symmetric(xx, y, a, b, use_epsilon_scaling=False, eps=eps,
                                         n_iters=2000)

    def loss(xx):
        f, g = potentials(xx)
        return gf @ f + gg @ g

    f, g = potentials(x)
    got = oracle.implicit_grad_x_from_potentials(
        x, y, f - (x ** 2).sum(1), g - (y ** 2).sum(1), gf, gg, eps=eps, log_a=np.log(a),
        log_b=np.log(b), tau2=1e-9)
    h = 1e-5
    for i in range(n):
        for k in range(d):
            xp, xm = x.copy(), x.copy()
            xp[i, k] += h; xm[i, k] -= h
            assert abs(got[i, k] - (loss(xp) - loss(xm)) / (2 * h)) < 1e-5 * (1 + abs(got[i, k]))


def test_inverse_hvp_inverts_the_hvp():
    rng = np.random.default_rng(1)
    n, m, d, eps = 7, 6, 2, 0.4
    x, y = rng.standard_normal((n, d)), rng.standard_normal((m, d))
    a, b = np.full(n, 1 / n), np.full(m, 1 / m)
    _, _, fp, gp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps,
                                             n_iters=50, return_prelast=True)
    fo, go = oracle.geomloss_to_ott_potentials(fp, gp, a, b, eps)
    gr = rng.standard_normal((n, d))
    z, H = oracle.inverse_hvp_x_from_potentials(x, y, fo, go, gr, eps=eps)
    back, _ = oracle.hvp_x_from_potentials(x, y, fo, go, z, eps=eps, max_cg_iter=2000,
                                           cg_rtol=1e-13, cg_atol=1e-14)
    np.testing.assert_allclose(back, gr, rtol=1e-7, atol=1e-9)
    np.testing.assert_allclose(H, H.T, rtol=1e-6, atol=1e-9)  # a Hessian


def test_c_transform_defining_properties():
    """c_i + psi_j <= C_ij for every j with equality at the returned index; nearest neighbour
    when psi = 0; the reference's tie construction resolves to the smaller index."""
    rng = np.random.default_rng(31)
    n, m, d, cs = 40, 57, 5, 0.5
    x, y, psi = rng.standard_normal((n, d)), rng.standard_normal((m, d)), rng.standard_normal(m)
    c, idx = oracle.c_transform(x, y, psi, cs)
    C = cs * ((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)
    assert np.all(c[:, None] + psi[None, :] <= C + 1e-12)
    np.testing.assert_allclose(c + psi[idx], C[np.arange(n), idx], rtol=0, atol=1e-12)
    c0, i0 = oracle.c_transform(x, x, np.zeros(n), 1.0)
    np.testing.assert_allclose(c0, 0.0, atol=1e-15)
    assert np.array_equal(i0, np.arange(n))
    # brute-force python loop
    for i in range(0, n, 7):
        best = min(range(m), key=lambda j: (cs * float(((x[i] - y[j]) ** 2).sum()) - psi[j], j))
        assert idx[i] == best
    # two equidistant targets: the smaller index wins (reference test_c_transform.py:179-213)
    yt = np.zeros((96, 4)); yt[:, 0] = 100.0; yt[0, 0] = 1.0; yt[64, 0] = -1.0
    _, it = oracle.c_transform(np.zeros((1, 4)), yt, np.zeros(96), 1.0)
    assert it[0] == 0


def test_c_transform_cost_gradients_by_finite_differences():
    rng = np.random.default_rng(32)
    n, m, d, cs = 12, 9, 3, 1.0
    x, y, psi = rng.standard_normal((n, d)), rng.standard_normal((m, d)), rng.standard_normal(m)
    a = rng.dirichlet(np.ones(n)); b = rng.dirichlet(np.ones(m))
    L, gx, gp, idx = oracle.c_transform_cost_grads(x, y, psi, a, b, cs)
    h = 1e-6  # far below the gap to the second-best target, so the minimiser does not move
    for (i, k) in [(0, 0), (5, 2), (11, 1)]:
        xp = x.copy(); xp[i, k] += h
        xm = x.copy(); xm[i, k] -= h
        fd = (oracle.c_transform_cost_grads(xp, y, psi, a, b, cs)[0]
              - oracle.c_transform_cost_grads(xm, y, psi, a, b, cs)[0]) / (2 * h)
        assert abs(fd - gx[i, k]) < 1e-6
    for j in [0, 4, 8]:
        pp = psi.copy(); pp[j] += h
        pm = psi.copy(); pm[j] -= h
        fd = (oracle.c_transform_cost_grads(x, y, pp, a, b, cs)[0]
              - oracle.c_transform_cost_grads(x, y, pm, a, b, cs)[0]) / (2 * h)
        assert abs(fd - gp[j]) < 1e-6
