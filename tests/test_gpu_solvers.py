"""Solvers, SamplesLoss, gradients and HVP on the GPU vs the oracle and golden vectors."""
import numpy as np
import pytest
import torch

import oracle
from tests.golden.recipe import inputs

pytestmark = pytest.mark.gpu
RTOL = 1e-4


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def rel_err(got, want):
    got = got.detach().cpu().numpy().astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def test_symmetric_solver_vs_reference_golden(golden):
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(11, 64, 48, 32)
    X, Y, A, B = dev(x, y, a, b)
    f, g, fp, gp = solve(X, Y, A, B, use_epsilon_scaling=False, eps=0.5, n_iters=3,
                         allow_tf32=False, return_prelast=True)
    assert rel_err(f, golden["sym_fixed_f"]) < RTOL and rel_err(g, golden["sym_fixed_g"]) < RTOL
    assert rel_err(fp, golden["sym_fixed_noext_f"]) < RTOL
    f, g = solve(X, Y, A, B, blur=0.5, scaling=0.7, allow_tf32=False)
    assert rel_err(f, golden["sym_scaling_f"]) < RTOL and rel_err(g, golden["sym_scaling_g"]) < RTOL
    f, g = solve(X, Y, A, B, use_epsilon_scaling=False, eps=0.05, n_iters=20, allow_tf32=False)
    # the golden vector is the reference's own fp32 torch run, 1.5e-4 from the fp64 answer at
    # this eps; against the fp64 oracle the bar is 1e-4
    assert rel_err(f, golden["sym_smalleps_f"]) < 2e-4
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.05, n_iters=20)
    assert rel_err(f, wf) < RTOL and rel_err(g, wg) < RTOL
    # fp16 inputs are cast to fp32 by the launchers (reference test uses fp16 x, y)
    f16, g16 = solve(X.half(), Y.half(), A, B, use_epsilon_scaling=False, eps=0.5, n_iters=3)
    assert rel_err(f16, golden["sym_fixed_f"]) < 2e-3  # the rounding of the inputs to fp16


def test_fused_equals_separate_and_exp2_flag():
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(31, 500, 420, 24)
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(use_epsilon_scaling=False, eps=0.2, n_iters=6, allow_tf32=False, reach_x=1.5)
    f1, g1 = solve(X, Y, A, B, fused=True, **kw)
    f2, g2 = solve(X, Y, A, B, fused=False, use_exp2=False, **kw)
    assert rel_err(f1, f2.cpu().numpy()) < 1e-5 and rel_err(g1, g2.cpu().numpy()) < 1e-5


@pytest.mark.parametrize("kw", [dict(reach=1.0), dict(reach_x=0.7), dict(rho_y=2.0),
                                dict(rho_x=0.5, rho_y=3.0)])
def test_unbalanced_symmetric_vs_oracle(kw):
    # parity unpinned by reference artefacts (its own tests need GeomLoss); pinned by restatement
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(32, 512, 300, 32, scale=0.5)
    a = a * 1.0; b = b * 1.3
    X, Y, A, B = dev(x, y, a, b)
    skw = dict(blur=0.3, scaling=0.6, cost_scale=0.5)
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, **skw, **kw)
    f, g = solve(X, Y, A, B, allow_tf32=False, **skw, **kw)
    assert rel_err(f, wf) < RTOL and rel_err(g, wg) < RTOL


@pytest.mark.parametrize("rx,ry", [(2.0, 0.7), (0.7, 2.0), (1.5, None), (None, 0.9)])
def test_unbalanced_symmetric_fixed_point_on_the_gpu(rx, ry):
    """No oracle involved: the GPU's unbalanced symmetric solver, run to its fixed point, returns
    potentials whose plan (its marginals taken with the GPU's plan-vector product) satisfies the
    first-order conditions of the KL-relaxed problem, P 1 = a exp(-f / rho_x) and
    P^T 1 = b exp(-g / rho_y), a balanced side meaning exp(.) = 1."""
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    from flash_sinkhorn_amd.kernels.apply_flash import apply_plan_vec_flashstyle as apply_vec
    x, y, a, b = inputs(33, 300, 260, 8, scale=0.5)
    b = (b * 1.3).astype(np.float32)
    eps = 0.5
    X, Y, A, B = dev(x, y, a, b)
    f, g = solve(X, Y, A, B, use_epsilon_scaling=False, eps=eps, n_iters=600, allow_tf32=False,
                 rho_x=rx, rho_y=ry)
    fh, gh = f - (X * X).sum(1), g - (Y * Y).sum(1)
    la, lb = torch.log(A), torch.log(B)
    row = apply_vec(X, Y, fh, gh, la, lb, torch.ones_like(B), eps=eps, axis=1)
    col = apply_vec(X, Y, fh, gh, la, lb, torch.ones_like(A), eps=eps, axis=0)
    want_row = A * (torch.exp(-f / rx) if rx is not None else 1.0)
    want_col = B * (torch.exp(-g / ry) if ry is not None else 1.0)
    assert float((row - want_row).abs().max()) < 1e-4 * float(want_row.max())
    assert float((col - want_col).abs().max()) < 1e-4 * float(want_col.max())


def test_alternating_solver(golden):
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_alternating as solve
    x, y, a, b = inputs(12, 40, 56, 16)
    X, Y, A, B = dev(x, y, a, b)
    f, g = solve(X, Y, A, B, eps=1.0, n_iters=5, ott_convention=True, allow_tf32=False)
    assert rel_err(f, golden["alt_ott_f"]) < RTOL and rel_err(g, golden["alt_ott_g"]) < RTOL
    # GeomLoss convention, unbalanced and semi-unbalanced, as the reference writes it
    for kw in (dict(), dict(reach=1.0), dict(reach_x=1.0, reach_y=None)):
        wf, wg, wn = oracle.sinkhorn_alternating(x, y, a, b, eps=0.3, n_iters=10, threshold=1e-3,
                                                 check_every=5, return_n_iters=True, **kw)
        f, g, n_used = solve(X, Y, A, B, eps=0.3, n_iters=10, threshold=1e-3, check_every=5,
                             return_n_iters=True, allow_tf32=False, **kw)
        assert n_used == wn and rel_err(f, wf) < RTOL and rel_err(g, wg) < RTOL


def test_early_stopping_counts_match_oracle():
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(33, 200, 180, 8)
    kw = dict(use_epsilon_scaling=False, eps=1.0, n_iters=60, threshold=1e-2, check_every=4,
              return_n_iters=True)
    *_, wn = oracle.sinkhorn_symmetric(x, y, a, b, **kw)
    *_, n_used = solve(*dev(x, y, a, b), allow_tf32=False, **kw)
    assert n_used == wn and n_used < 62


def test_warm_start():
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(34, 100, 90, 8)
    rng = np.random.default_rng(1)
    f0 = rng.standard_normal(100).astype(np.float32); g0 = rng.standard_normal(90).astype(np.float32)
    kw = dict(use_epsilon_scaling=False, eps=0.5, n_iters=2)
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, f_init=f0, g_init=g0, **kw)
    X, Y, A, B, F0, G0 = dev(x, y, a, b, f0, g0)
    f, g = solve(X, Y, A, B, f_init=F0, g_init=G0, allow_tf32=False, **kw)
    assert rel_err(f, wf) < RTOL and rel_err(g, wg) < RTOL


def _loss_oracle(x, y, a, b, *, eps, n_iters, cost_scale, debias):
    def ot(x1, y1, a1, b1):
        f, g, fp, gp = oracle.sinkhorn_symmetric(x1, y1, a1, b1, use_epsilon_scaling=False,
                                                 eps=eps, n_iters=n_iters, cost_scale=cost_scale,
                                                 return_prelast=True)
        gx, gy = oracle.grad_barycentric(x1, y1, a1, b1, fp, gp, eps, cost_scale)
        return oracle.sinkhorn_cost(a1, b1, f, g, eps), gx, gy
    c, gx, _ = ot(x, y, a, b)
    if debias:
        cxx, gxx_x, gxx_y = ot(x, x, a, a)
        cyy, _, _ = ot(y, y, b, b)
        c = c - 0.5 * cxx - 0.5 * cyy
        gx = gx - 0.5 * (gxx_x + gxx_y)  # x feeds both clouds of OT(x, x)
    return c, gx


def test_samples_loss_value_and_gradient_config1_shape():
    # benchmark configuration 1 at reduced n: debiased, half cost, eps=0.01, d=3, uniform weights
    from flash_sinkhorn_amd import SamplesLoss
    rng = np.random.default_rng(1)
    n = m = 400
    x = rng.standard_normal((n, 3)).astype(np.float32)
    y = rng.standard_normal((m, 3)).astype(np.float32)
    a = np.full(n, 1 / n, np.float32); b = np.full(m, 1 / m, np.float32)
    want, want_gx = _loss_oracle(x, y, a, b, eps=0.01, n_iters=100, cost_scale=0.5, debias=True)
    X = torch.from_numpy(x).cuda().requires_grad_(True)
    Y = torch.from_numpy(y).cuda()
    loss = SamplesLoss("sinkhorn", blur=0.1, half_cost=True, debias=True,
                       use_epsilon_scaling=False, eps=0.01, n_iters=100, allow_tf32=False)(X, Y)
    (gx,) = torch.autograd.grad(loss, X)
    assert abs(float(loss) - want) <= 1e-4 * max(abs(want), 1e-3) + 2e-6
    assert rel_err(gx, want_gx) < RTOL


def test_samples_loss_api_forms():
    from flash_sinkhorn_amd import SamplesLoss
    x, y, a, b = inputs(35, 150, 130, 5, uniform=True)
    X, Y, A, B = dev(x, y, a, b)
    L = SamplesLoss(blur=0.3, allow_tf32=False)
    c1, c2 = L(X, Y), L(A, X, B, Y)
    assert abs(float(c1) - float(c2)) < 1e-6 * abs(float(c1)) + 1e-7
    f, g = SamplesLoss(blur=0.3, potentials=True, allow_tf32=False)(A[:, None], X, B, Y)
    assert f.shape == (150, 1) and g.shape == (130,)
    assert abs(float((A * f[:, 0]).sum() + (B * g).sum()) - float(c1)) < 1e-5 * abs(float(c1))
    cb = L(torch.stack([X, X]), torch.stack([Y, Y]))
    assert cb.shape == (2,) and abs(float(cb[1]) - float(c1)) < 1e-6 * abs(float(c1)) + 1e-7
    z = SamplesLoss(blur=0.3, debias=True, allow_tf32=False)(X, X)
    assert abs(float(z)) < 1e-5
    half = SamplesLoss(blur=0.3, half_cost=True, allow_tf32=False)(X, Y)
    want_half = oracle.sinkhorn_cost(a, b, *oracle.sinkhorn_symmetric(
        x, y, a, b, blur=0.3, cost_scale=0.5), 0.09)
    assert abs(float(half) - want_half) < 1e-4 * abs(want_half)
    alt = SamplesLoss(backend="alternating", use_epsilon_scaling=False, eps=0.2, n_iters=8,
                      allow_tf32=False)(X, Y)
    wf, wg = oracle.sinkhorn_alternating(x, y, a, b, eps=0.2, n_iters=8)
    assert abs(float(alt) - oracle.sinkhorn_cost(a, b, wf, wg, 0.2)) < 1e-4 * abs(float(alt))
    unb = SamplesLoss(blur=0.3, reach=1.0, allow_tf32=False)(X, Y)
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, blur=0.3, reach=1.0)
    want = oracle.sinkhorn_cost(a, b, wf, wg, 0.09, rho_x=1.0, rho_y=1.0)
    assert abs(float(unb) - want) < 1e-4 * abs(want)


def test_hvp_vs_reference_golden_and_oracle(golden):
    from flash_sinkhorn_amd import hvp_x_sqeuclid_from_potentials as hvp
    x, y, a, b = inputs(13, 32, 24, 8)
    A, f, g = golden["hvp_A"], golden["hvp_f_ott"], golden["hvp_g_ott"]
    X, Y, F, G, AA = dev(x, y, f, g, A)
    h, info = hvp(X, Y, F, G, AA, eps=0.2)
    # the balanced Schur system is the worst conditioned of the four: an fp32 CG solve lands
    # 1.3e-4 from the fp64 dense solve, here (1.3e-4) as in the reference's own fp32 run that
    # wrote the golden vector (1.4e-4); the relaxed variants below meet 1e-4
    assert rel_err(h, golden["hvp_plain"]) < 2e-4 and info.cg_converged
    want, _ = oracle.hvp_x_from_potentials(x, y, f, g, A, eps=0.2)
    assert rel_err(h, want) < 2e-4
    for tag, rx, ry in (("hvp_semi_x", 1.0, None), ("hvp_semi_y", None, 0.5),
                        ("hvp_unbal", 1.0, 2.0)):
        h, info = hvp(X, Y, F, G, AA, eps=0.2, rho_x=rx, rho_y=ry)
        assert rel_err(h, golden[tag]) < RTOL
    # half cost and the preconditioned operator: restatement only (see oracle header)
    want, _ = oracle.hvp_x_from_potentials(x, y, f, g, A, eps=0.2, cost_scale=0.5,
                                           preconditioner="jacobi")
    h, _ = hvp(X, Y, F, G, AA, eps=0.2, cost_scale=0.5, preconditioner="jacobi")
    assert rel_err(h, want) < RTOL
    psd, ind, _ = hvp(X, Y, F, G, AA, eps=0.2, return_components=True)
    assert rel_err(psd + ind, golden["hvp_plain"]) < 2e-4  # fp32 golden, as above


def test_double_backward_equals_direct_hvp():
    from flash_sinkhorn_amd import (SamplesLoss, geomloss_to_ott_potentials,
                                    hvp_x_sqeuclid_from_potentials)
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, y, a, b = inputs(36, 96, 80, 6)
    v = np.random.default_rng(2).standard_normal(x.shape).astype(np.float32)
    X, Y, A, B, V = dev(x, y, a, b, v)
    X.requires_grad_(True)
    L = SamplesLoss(use_epsilon_scaling=False, eps=0.3, n_iters=30, allow_tf32=False,
                    half_cost=True)
    (gx,) = torch.autograd.grad(L(A, X, B, Y), X, create_graph=True)
    (hv,) = torch.autograd.grad((gx * V).sum(), X)
    _, _, fp, gp = solve(X.detach(), Y, A, B, use_epsilon_scaling=False, eps=0.3, n_iters=30,
                         allow_tf32=False, cost_scale=0.5, return_prelast=True)
    fo, go = geomloss_to_ott_potentials(fp, gp, A, B, eps=0.3)
    want, _ = hvp_x_sqeuclid_from_potentials(X.detach(), Y, fo, go, V, eps=0.3, cost_scale=0.5)
    assert rel_err(hv, want.cpu().numpy()) < 1e-5
    with pytest.raises(NotImplementedError):
        Yg = Y.clone().requires_grad_(True)
        gx, gy = torch.autograd.grad(L(A, X, B, Yg), [X, Yg], create_graph=True)
        torch.autograd.grad((gy * gy).sum(), Yg)


@pytest.mark.parametrize("kw", [dict(), dict(reach=0.8)])
def test_self_problem_shortcut_equals_generic_path(kw):
    """OT(x, x) with aliased arguments runs one half-update per step; a copy of x (no
    aliasing) takes the two-sided path.  Same numbers either way."""
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric as solve
    x, _, a, _ = inputs(37, 700, 700, 16)
    X, A = dev(x, a)
    args = dict(use_epsilon_scaling=False, eps=0.05, n_iters=20, allow_tf32=False,
                return_prelast=True, **kw)
    fs, gs, fps, gps = solve(X, X, A, A, **args)
    fg, gg, fpg, gpg = solve(X, X.clone(), A, A.clone(), **args)
    assert torch.equal(fs, gs) and torch.equal(fps, gps)
    assert float((fs - fg).abs().max()) <= 1e-6 * float(fg.abs().max())
    assert float((gs - gg).abs().max()) <= 1e-6 * float(gg.abs().max())
    assert float((fps - fpg).abs().max()) <= 1e-6 * float(fpg.abs().max())
    want = oracle.sinkhorn_symmetric(x, x, a, a, use_epsilon_scaling=False, eps=0.05, n_iters=20,
                                     **kw)
    assert rel_err(fs, want[0]) < RTOL and rel_err(gs, want[1]) < RTOL


@pytest.mark.parametrize("n,m,d", [(700, 500, 64), (300, 260, 200)])
def test_prepared_operands_give_identical_results(n, m, d):
    """Planes written once by fs_prepare_operands serve the symmetric step and both roles of
    the one-sided LSE; results are bit-identical to calls that convert their operands."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        _symmetric_step_raw, flashsinkhorn_lse_fused)
    x, y, a, b = inputs(41, n, m, d, scale=2.0 / np.sqrt(d))
    rng = np.random.default_rng(3)
    fh = (rng.standard_normal(n) * 0.3).astype(np.float32)
    gh = (rng.standard_normal(m) * 0.3).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, np.log(a), np.log(b))
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    f0, g0 = _symmetric_step_raw(X, Y, F, G, LA, LB, 0.2, **kw)
    f1, g1 = _symmetric_step_raw(X, Y, F, G, LA, LB, 0.2, prepared=prep, **kw)
    assert torch.equal(f0, f1) and torch.equal(g0, g1)
    for q, k, pot, lw in ((X, Y, G, LB), (Y, X, F, LA)):
        o0 = flashsinkhorn_lse_fused(q, k, pot, lw, 0.2, allow_tf32=False)
        o1 = flashsinkhorn_lse_fused(q, k, pot, lw, 0.2, allow_tf32=False, _prepared=prep)
        assert torch.equal(o0, o1)
    # allow_tf32=True is served by the same planes
    o2 = flashsinkhorn_lse_fused(X, Y, G, LB, 0.2, allow_tf32=True, _prepared=prep)
    assert torch.equal(o2, flashsinkhorn_lse_fused(X, Y, G, LB, 0.2, allow_tf32=False))

@pytest.mark.parametrize("n,m,d", [(3000, 4100, 64), (129, 1000, 3), (5000, 300, 128), (260, 260, 32)])
def test_launches_are_repeatable_on_one_workspace(n, m, d, monkeypatch):
    """Split keys leave partial rows in the workspace between the streaming kernel and the merge:
    every launch on one prepared workspace must give the bits of the first, and of a call with
    a fresh workspace (nothing carried over, no dependence on workgroup arrival order).  The one
    thing that is carried on purpose, the permission to take both sides from one sweep, is
    switched off for that and looked at afterwards: with it, launches on the same inputs give the
    two-sided kernel's bits until the form is on, the same bits as each other from then on, and
    the two-sided kernel's numbers to rounding."""
    from flash_sinkhorn_amd import _lib
    monkeypatch.setattr(_lib, "SWEEP", False)
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    x, y, a, b = inputs(47, n, m, d, scale=2.0 / np.sqrt(d))
    rng = np.random.default_rng(5)
    fh = (rng.standard_normal(n) * 0.3).astype(np.float32)
    gh = (rng.standard_normal(m) * 0.3).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, np.log(a), np.log(b))
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    f0, g0 = _symmetric_step_raw(X, Y, F, G, LA, LB, 0.2, **kw)
    wf, wg = oracle.symmetric_step(x, y, fh, gh, np.log(a), np.log(b), 0.2, 1.0, 0.5, 1.0, 1.0)
    assert rel_err(f0, wf) < RTOL and rel_err(g0, wg) < RTOL
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    for _ in range(25):
        f1, g1 = _symmetric_step_raw(X, Y, F, G, LA, LB, 0.2, prepared=prep, **kw)
        assert torch.equal(f0, f1) and torch.equal(g0, g1)
    monkeypatch.setattr(_lib, "SWEEP", True)
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    later = []
    for it in range(12):
        on = prep.variant_state()["sweep_next"]
        f1, g1 = _symmetric_step_raw(X, Y, F, G, LA, LB, 0.2, prepared=prep, **kw)
        if not on:
            assert torch.equal(f0, f1) and torch.equal(g0, g1)
        else:
            later.append((f1, g1))
            assert torch.equal(later[0][0], f1) and torch.equal(later[0][1], g1)
            assert rel_err(f1, f0.cpu().numpy()) < 2e-6 and rel_err(g1, g0.cpu().numpy()) < 2e-6
    assert (len(later) > 0) == (min(n, m) >= 2048 and d <= 64)
    monkeypatch.setattr(_lib, "SWEEP", False)
    if n == m:  # the aliased self problem on its own prepared workspace
        s0, _ = _symmetric_step_raw(X, X, F, F, LA, LA, 0.2, **kw)
        prep = _lib.PreparedOperands(X, X, _lib.flags(True, False))
        for _ in range(10):
            s1, _ = _symmetric_step_raw(X, X, F, F, LA, LA, 0.2, prepared=prep, **kw)
            assert torch.equal(s0, s1)


@pytest.mark.parametrize("n,m,d", [(700, 500, 64), (300, 260, 200)])
def test_multi_step_call_equals_single_steps(n, m, d):
    """fs_symmetric_steps enqueues the same launches as a loop over fs_symmetric_step: the
    potentials are bit-identical, for a schedule with changing eps, weights and dampings, for
    odd and even step counts, and for the aliased self problem."""
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        _symmetric_step_raw, _symmetric_steps_raw)
    x, y, a, b = inputs(43, n, m, d, scale=2.0 / np.sqrt(d))
    X, Y, LA, LB = dev(x, y, np.log(a), np.log(b))
    AL, BE = (X * X).sum(1).contiguous(), (Y * Y).sum(1).contiguous()
    steps = [(0.8, 1.0, 1.0, 1.0), (0.5, 0.5, 0.9, 0.8), (0.3, 0.5, 0.9, 0.8),
             (0.2, 0.5, 0.95, 0.85), (0.2, 1.0, 0.95, 0.85)]
    for k in (1, 4, 5):
        f, g = -AL, -BE
        for e, w, df, dg in steps[:k]:
            f, g = _symmetric_step_raw(X, Y, f, g, LA, LB, e, cost_scale=1.0, alpha=w,
                                       damping_f=df, damping_g=dg, shift_x=AL, shift_y=BE,
                                       allow_tf32=False)
        f2, g2 = _symmetric_steps_raw(X, Y, -AL, -BE, LA, LB, steps[:k], cost_scale=1.0,
                                      shift_x=AL, shift_y=BE, allow_tf32=False)
        assert torch.equal(f, f2) and torch.equal(g, g2)
    # self problem: one half-update per step, one tensor returned twice
    f0 = -AL
    sym = [(e, w, df, df) for e, w, df, _ in steps]
    f, g = f0, f0
    for e, w, df, _ in sym:
        f, g = _symmetric_step_raw(X, X, f, g, LA, LA, e, cost_scale=1.0, alpha=w, damping_f=df,
                                   damping_g=df, shift_x=AL, shift_y=AL, allow_tf32=False)
    f2, g2 = _symmetric_steps_raw(X, X, f0, f0, LA, LA, sym, cost_scale=1.0, shift_x=AL,
                                  shift_y=AL, allow_tf32=False)
    assert f2 is g2 and torch.equal(f, f2)


def test_inverse_hvp_against_dense_oracle():
    """Outer CG on the streaming HVP against a dense solve with the oracle's Hessian."""
    from flash_sinkhorn_amd import (geomloss_to_ott_potentials, hvp_x_sqeuclid_from_potentials,
                                    inverse_hvp_x_sqeuclid_from_potentials)
    rng = np.random.default_rng(5)
    n, m, d, eps = 12, 10, 3, 0.4
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = rng.standard_normal((m, d)).astype(np.float32)
    a, b = np.full(n, 1 / n, np.float32), np.full(m, 1 / m, np.float32)
    _, _, fp, gp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps,
                                             n_iters=40, return_prelast=True)
    fo, go = oracle.geomloss_to_ott_potentials(fp, gp, a, b, eps)
    gr = rng.standard_normal((n, d)).astype(np.float32)
    want, H = oracle.inverse_hvp_x_from_potentials(x, y, fo, go, gr, eps=eps)
    X, Y, FO, GO, GR = dev(x, y, fo.astype(np.float32), go.astype(np.float32), gr)
    z, info = inverse_hvp_x_sqeuclid_from_potentials(X, Y, FO, GO, GR, eps=eps)
    # fp32 CG on a system of condition number cond(H): the bar scales with it
    cond = np.linalg.cond(H)
    assert rel_err(z, want) < max(2e-3, 1e-6 * cond)
    back, _ = hvp_x_sqeuclid_from_potentials(X, Y, FO, GO, z, eps=eps)
    assert rel_err(back, gr) < 1e-3


@pytest.mark.parametrize("cs", [1.0, 0.5])
def test_implicit_gradient_against_oracle(cs):
    from flash_sinkhorn_amd import implicit_grad_x, implicit_grad_x_from_potentials
    x, y, a, b = inputs(71, 300, 260, 6)
    rng = np.random.default_rng(6)
    gf = rng.standard_normal(300).astype(np.float32)
    gg = rng.standard_normal(260).astype(np.float32)
    eps = 0.3
    f, g = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=eps, n_iters=60,
                                     cost_scale=cs)
    fh = f - cs * (x.astype(np.float64) ** 2).sum(1)
    gh = g - cs * (y.astype(np.float64) ** 2).sum(1)
    want = oracle.implicit_grad_x_from_potentials(x, y, fh, gh, gf, gg, eps=eps, log_a=np.log(a),
                                                  log_b=np.log(b), cost_scale=cs)
    X, Y, A, B, FH, GH, GF, GG = dev(x, y, a, b, fh.astype(np.float32), gh.astype(np.float32),
                                     gf, gg)
    got, info = implicit_grad_x_from_potentials(X, Y, FH, GH, GF, GG, eps=eps, log_a=A.log(),
                                                log_b=B.log(), cost_scale=cs, max_cg_iter=300)
    assert info.cg_converged and rel_err(got, want) < 2e-3
    got2, _ = implicit_grad_x(X, Y, A, B, GF, GG, eps=eps, cost_scale=cs, n_iters=60,
                              max_cg_iter=300)
    assert rel_err(got2, want) < 2e-3


def test_custom_operators_match_the_launchers():
    """torch.ops.flash_sinkhorn_amd.* run the same library calls as the launchers they wrap."""
    from flash_sinkhorn_amd import torch_ops  # noqa: F401  (registers the operators)
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_lse_fused, flashsinkhorn_symmetric_step)
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    ops = torch.ops.flash_sinkhorn_amd
    n, m, d = 300, 260, 40
    x, y, a, b = inputs(47, n, m, d, scale=2.0 / np.sqrt(d))
    rng = np.random.default_rng(4)
    fh = (rng.standard_normal(n) * 0.3).astype(np.float32)
    gh = (rng.standard_normal(m) * 0.3).astype(np.float32)
    X, Y, A, B, F, G, LA, LB = dev(x, y, a, b, fh, gh, np.log(a), np.log(b))
    assert torch.equal(ops.lse_fused(X, Y, G, LB, 0.2),
                       flashsinkhorn_lse_fused(X, Y, G, LB, 0.2, allow_tf32=False))
    f1, g1 = ops.symmetric_step(X, Y, F, G, LA, LB, 0.2)
    f2, g2 = flashsinkhorn_symmetric_step(X, Y, F, G, LA, LB, 0.2, allow_tf32=False)
    assert torch.equal(f1, f2) and torch.equal(g1, g2)
    gx1, gy1 = ops.grad(X, Y, A, B, F, G, 0.2, 0.5)
    gx2, gy2 = grad(X, Y, A, B, F, G, eps=0.2, cost_scale=0.5, allow_tf32=False)
    assert torch.equal(gx1, gx2) and torch.equal(gy1, gy2)
    v = torch.randn(m, device="cuda")
    V = torch.randn(m, d, device="cuda")
    assert torch.equal(ops.apply_plan_vec(X, Y, F, G, LA, LB, v, 0.4, 1),
                       apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, v, eps=0.4, axis=1))
    assert torch.equal(ops.apply_plan_mat(X, Y, F, G, LA, LB, V, 0.4, 1),
                       apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, V, eps=0.4, axis=1))
    c, idx = ops.c_transform(X, Y, (Y * Y).sum(1) - G)
    want_c, want_idx = oracle.c_transform(x, y, gh, 1.0)
    inner = want_c - (x.astype(np.float64) ** 2).sum(1)
    assert np.abs(c.cpu().numpy() - inner).max() <= 1e-5 * np.abs(inner).max()
    assert (idx.cpu().numpy() == want_idx).mean() > 0.99
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_fused_sqeuclid import (
        fused_schur_matvec_sqeuclid)
    dx, dn = torch.rand(n, device="cuda") + 0.5, torch.rand(m, device="cuda") + 0.5
    o1, p1 = ops.schur_matvec(X, Y, F, G, v, dx, dn, 0.4)
    o2, p2 = fused_schur_matvec_sqeuclid(X, Y, F, G, v, dx, dn, eps=0.4)
    assert torch.equal(o1, o2) and torch.equal(p1, p2)
    torch.library.opcheck(ops.lse_fused.default, (X, Y, G, LB, 0.2),
                          test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("n,m,d", [(700, 500, 64), (300, 260, 200), (2000, 2000, 3)])
@pytest.mark.parametrize("kw", [
    dict(use_epsilon_scaling=False, eps=0.1, n_iters=12),
    dict(use_epsilon_scaling=False, eps=0.1, n_iters=7, last_extrapolation=False),
    dict(use_epsilon_scaling=True, blur=0.3, scaling=0.7),
    dict(use_epsilon_scaling=True, blur=0.3, scaling=0.7, rho=2.0),
])
def test_self_pair_equals_separate_self_solves(n, m, d, kw):
    """The two debiasing self problems advanced in shared launches (fs_self_pair_steps) give
    the potentials of the two independent self solves; under eps-scaling the clouds have
    different diameters, hence schedules of different lengths."""
    from flash_sinkhorn_amd.sinkhorn_solvers import (
        sinkhorn_flashstyle_symmetric, sinkhorn_flashstyle_symmetric_self_pair)
    x, y, a, b = inputs(61, n, m, d, scale=1.0 / np.sqrt(d))
    y = (y * 2.5).astype(np.float32)          # a wider cloud: a longer eps schedule
    X, Y, A, B = dev(x, y, a, b)
    solo = dict(kw)
    rho = solo.pop("rho", None)
    last = kw.get("last_extrapolation", True)
    out_x, out_y = sinkhorn_flashstyle_symmetric_self_pair(
        X, A, Y, B, allow_tf32=False, return_prelast=True, **kw)
    for pts, w, got in ((X, A, out_x), (Y, B, out_y)):
        want = sinkhorn_flashstyle_symmetric(pts, pts, w, w, allow_tf32=False, rho_x=rho,
                                             rho_y=rho, return_prelast=True, **solo)
        assert len(got) == len(want) == (4 if last else 2)
        for g, wv in zip(got, want):
            scale = float(wv.abs().max())
            assert float((g - wv).abs().max()) <= 2e-6 * scale


def test_debiased_loss_with_paired_self_terms_equals_separate(monkeypatch):
    """SamplesLoss(debias=True) solves its two self terms together; loss and gradients equal
    those of the three independent solves."""
    import flash_sinkhorn_amd.samples_loss as sl
    from flash_sinkhorn_amd import SamplesLoss
    x, y, a, b = inputs(63, 900, 700, 8, scale=0.5)
    for cfg in (dict(blur=0.1, use_epsilon_scaling=False, eps=0.01, n_iters=20),
                dict(blur=0.2, scaling=0.6), dict(blur=0.2, scaling=0.6, reach=1.5)):
        results = []
        for paired in (True, False):
            X, Y, A, B = dev(x, y, a, b)
            X.requires_grad_(True)
            Y.requires_grad_(True)
            loss_fn = SamplesLoss("sinkhorn", debias=True, allow_tf32=False, **cfg)
            if not paired:
                loss_fn.threshold = 1e-30      # never met: switches the pairing off only
            val = loss_fn(A, X, B, Y)
            gx, gy = torch.autograd.grad(val, [X, Y])
            results.append((val.detach(), gx, gy))
        (v1, gx1, gy1), (v0, gx0, gy0) = results
        assert abs(float(v1 - v0)) <= 1e-5 * max(abs(float(v0)), 1e-3)
        assert float((gx1 - gx0).abs().max()) <= 1e-5 * float(gx0.abs().max())
        assert float((gy1 - gy0).abs().max()) <= 1e-5 * float(gy0.abs().max())


def test_debiased_loss_side_stream_matches_single_stream(monkeypatch):
    """The self terms of a debiased loss run on a second stream; loss and gradient are those of
    the single-stream path bit for bit, also when the loss is called repeatedly (the allocator
    must not hand the side stream's results out again while they are in use)."""
    import flash_sinkhorn_amd.samples_loss as sl
    from flash_sinkhorn_amd import SamplesLoss
    x, y, a, b = inputs(67, 1500, 1300, 16, scale=0.4)
    loss_fn = SamplesLoss("sinkhorn", debias=True, allow_tf32=False, blur=0.1,
                          use_epsilon_scaling=False, eps=0.01, n_iters=30)

    def run():
        X, Y, A, B = dev(x, y, a, b)
        X.requires_grad_(True)
        v = loss_fn(A, X, B, Y)
        g, = torch.autograd.grad(v, [X])
        return v.detach().clone(), g.clone()

    monkeypatch.setattr(sl, "DEBIAS_SIDE_STREAM", False)
    v0, g0 = run()
    monkeypatch.setattr(sl, "DEBIAS_SIDE_STREAM", True)
    for _ in range(6):
        v1, g1 = run()
        junk = [torch.randn(1500, 16, device="cuda") for _ in range(4)]  # allocator churn
        assert torch.equal(v0, v1) and torch.equal(g0, g1)
        del junk


@pytest.mark.parametrize("m,every", [(300, 1), (300, 4), (5000, 3), (70000, 2)])
def test_device_cg_matches_host_cg(m, every):
    """fs_cg_init / fs_cg_update against the PyTorch-op CG on a dense SPD system: same
    solution, same convergence flag and iteration count, also when several iterations are
    enqueued between two looks at the state; non-convergence and zero right-hand sides follow
    the same conventions."""
    from flash_sinkhorn_amd.cg import conjugate_gradient, conjugate_gradient_device
    g = torch.Generator(device="cpu").manual_seed(m)
    k = 40
    U = torch.randn(m, k, generator=g).cuda() / np.sqrt(k)
    dvec = (1.0 + torch.rand(m, generator=g)).cuda()
    b = torch.randn(m, generator=g).cuda()

    def matvec(v):
        return dvec * v + U @ (U.t() @ v)

    want, wi = conjugate_gradient(matvec, b, max_iter=200, rtol=1e-6, atol=1e-10)
    got, gi = conjugate_gradient_device(matvec, b, max_iter=200, rtol=1e-6, atol=1e-10,
                                        check_every=every)
    assert wi.cg_converged and gi.cg_converged
    assert abs(gi.cg_iters - wi.cg_iters) <= 1
    assert float((got - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert abs(gi.cg_initial_residual - wi.cg_initial_residual) <= 1e-5 * wi.cg_initial_residual
    assert gi.cg_residual <= max(1e-10, 1e-6 * gi.cg_initial_residual)
    # too few iterations: not converged, the count is the limit
    _, g2 = conjugate_gradient_device(matvec, b, max_iter=2, rtol=1e-12, atol=0.0,
                                      check_every=every)
    _, w2 = conjugate_gradient(matvec, b, max_iter=2, rtol=1e-12, atol=0.0)
    assert (g2.cg_converged, g2.cg_iters) == (w2.cg_converged, w2.cg_iters) == (False, 2)
    assert abs(g2.cg_residual - w2.cg_residual) <= 1e-4 * w2.cg_residual
    # zero right-hand side: zero curvature ends the loop, solution zero
    z, g3 = conjugate_gradient_device(matvec, torch.zeros_like(b), max_iter=5, check_every=every)
    assert float(z.abs().max()) == 0.0 and not g3.cg_converged and g3.cg_iters == 5


@pytest.mark.parametrize("n,m,d", [(300, 257, 64), (129, 1000, 3), (100, 1100, 300),
                                   (2100, 2300, 20), (257, 300, 128)])
@pytest.mark.parametrize("cs", [1.0, 0.5])
def test_fused_schur_matvec_against_dense_oracle(n, m, d, cs):
    """out = denom*z - P^T((P z)/diag_x) with OTT potentials, P = exp((f+g-C)/eps): the two
    launches with their element-wise factors in the epilogues against the dense fp64 product;
    the returned buffer holds (P z)/diag_x and is reused when passed back."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_fused_sqeuclid import (
        fused_schur_matvec_sqeuclid)
    x, y, a, b = inputs(71, n, m, d, scale=2.0 / np.sqrt(d))
    rng = np.random.default_rng(13)
    eps = 0.4
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    C = cs * ((x64[:, None, :] - y64[None, :, :]) ** 2).sum(-1)
    f = (rng.standard_normal(n) * 0.2 + eps * np.log(a) - 1.0).astype(np.float32)
    g = (rng.standard_normal(m) * 0.2 + eps * np.log(b)).astype(np.float32)
    P = np.exp((f.astype(np.float64)[:, None] + g.astype(np.float64)[None, :] - C) / eps)
    z = rng.standard_normal(m).astype(np.float32)
    diag_x = (P.sum(1) * (1.0 + rng.random(n))).astype(np.float32)
    denom = (P.sum(0) * (1.0 + rng.random(m)) + 1e-3).astype(np.float32)
    piz_want = (P @ z.astype(np.float64)) / diag_x.astype(np.float64)
    want = denom.astype(np.float64) * z - P.T @ piz_want
    X, Y, F, G, Z, DX, DN = dev(x, y, f, g, z, diag_x, denom)
    out, piz = fused_schur_matvec_sqeuclid(X, Y, F, G, Z, DX, DN, eps=eps, cost_scale=cs)
    assert rel_err(piz, piz_want) < RTOL
    assert float(np.abs(out.cpu().numpy() - want).max()) <= RTOL * max(
        np.abs(denom * z).max(), np.abs(P.T @ piz_want).max())
    out2, piz2 = fused_schur_matvec_sqeuclid(X, Y, F, G, Z, DX, DN, eps=eps, cost_scale=cs,
                                             piz_buffer=piz)
    assert piz2 is piz and torch.equal(out, out2)
    with pytest.raises(ValueError):
        fused_schur_matvec_sqeuclid(X, Y, F, G, Z[:-1], DX, DN, eps=eps)
    with pytest.raises(ValueError):
        fused_schur_matvec_sqeuclid(X, Y, F, G, Z, DX[:-1], DN, eps=eps)


def _clustered(rng, n, d, k=8, spread=2.0):
    centres = rng.standard_normal((k, d)) * spread
    lab = rng.integers(0, k, n)
    return (centres[lab] + rng.standard_normal((n, d))).astype(np.float32), lab


@pytest.mark.parametrize("n,m,d,eps,sort", [(3000, 4100, 64, 0.01, True), (3000, 4100, 64, 0.01, False),
                                            (2100, 2300, 20, 0.3, False), (129, 1000, 3, 0.05, True),
                                            (40, 33, 16, 0.5, False), (2500, 3100, 128, 0.02, True),
                                            (1100, 2300, 100, 0.3, False), (70, 200, 65, 0.1, False)])
def test_coarse_tile_test_leaves_results_unchanged(n, m, d, eps, sort):
    """FS_FLAG_COARSE_TEST (tiles tested after their hi*hi plane product, running maximum started
    from 64 sampled keys) against the oracle and against the launch without the flag, on peaked
    plans over rows sorted by cluster (most tiles end at the test) and on generic inputs."""
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    rng = np.random.default_rng(31)
    x, lx = _clustered(rng, n, d)
    y, ly = _clustered(rng, m, d)
    if sort:
        x, y = x[np.argsort(lx, kind="stable")], y[np.argsort(ly, kind="stable")]
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    fh = (-(x * x).sum(1) + 0.1 * rng.standard_normal(n)).astype(np.float32)
    gh = (-(y * y).sum(1) + 0.1 * rng.standard_normal(m)).astype(np.float32)
    la, lb = np.log(a), np.log(b)
    args = dev(x, y, fh, gh, la, lb)
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    f1, g1 = _symmetric_step_raw(*args, eps, coarse=True, **kw)
    f0, g0 = _symmetric_step_raw(*args, eps, coarse=False, **kw)
    wf, wg = oracle.symmetric_step(x, y, fh, gh, la, lb, eps, 1.0, 0.5, 1.0, 1.0)
    assert rel_err(f1, wf) < RTOL and rel_err(g1, wg) < RTOL
    # the two launches differ by the order of the plane products only
    assert rel_err(f1, f0.cpu().numpy()) < 2e-6 and rel_err(g1, g0.cpu().numpy()) < 2e-6


@pytest.mark.parametrize("n,m,d,eps", [(3000, 4100, 64, 0.01), (2100, 2300, 20, 0.3), (700, 5000, 33, 0.02),
                                       (2200, 3300, 128, 0.02), (900, 2600, 80, 0.1)])
def test_coarse_test_starts_rows_from_the_keys_of_the_last_step(n, m, d, eps):
    """On prepared planes the kernel with the coarse tile test keeps, per row, the key that held
    the row's largest logit, and starts the next launch from the row's current logit at that key.
    After one step the kept keys are the arg-max keys; a step on very different potentials, and
    one on a key array overwritten with arbitrary numbers (negative, past the key set), still
    equal the oracle and the plain launch: any key gives a lower bound of the row's maximum."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    rng = np.random.default_rng(36)
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    a = np.full(n, 1.0 / n, np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    b /= b.sum()
    la, lb = np.log(a), np.log(b)
    fh = (-(x * x).sum(1) + 0.1 * rng.standard_normal(n)).astype(np.float32)
    gh = (-(y * y).sum(1) + 0.1 * rng.standard_normal(m)).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    kx, ky = prep.best_keys(0), prep.best_keys(1)
    assert int(kx.max()) == -1 and int(ky.max()) == -1
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)

    def check(f_in, g_in, F_in, G_in):
        f1, g1 = _symmetric_step_raw(X, Y, F_in, G_in, LA, LB, eps, coarse=True, prepared=prep, **kw)
        f0, g0 = _symmetric_step_raw(X, Y, F_in, G_in, LA, LB, eps, coarse=False, prepared=prep, **kw)
        wf, wg = oracle.symmetric_step(x, y, f_in, g_in, la, lb, eps, 1.0, 0.5, 1.0, 1.0)
        assert rel_err(f1, wf) < RTOL and rel_err(g1, wg) < RTOL
        assert rel_err(f1, f0.cpu().numpy()) < 2e-6 and rel_err(g1, g0.cpu().numpy()) < 2e-6

    check(fh, gh, F, G)
    # every row has a key now, and it is the arg-max key (ties and near-ties aside)
    logits = (2.0 * x.astype(np.float64) @ y.astype(np.float64).T + gh[None, :]) / eps + lb[None, :]
    kxh = kx.cpu().numpy()
    assert kxh.min() >= 0 and kxh.max() < m
    assert np.mean(kxh == logits.argmax(1)) > 0.97
    top = logits.max(1)
    assert np.all(logits[np.arange(n), kxh] > top - 1e-3 * np.abs(top).max())
    assert int(ky.min()) >= 0 and int(ky.max()) < n
    before = prep.variant_state()["tiles_tested"]
    # potentials far from the last step's: the kept keys are stale, their logits still bound the maxima
    fh2 = (fh + 3.0 * rng.standard_normal(n)).astype(np.float32)
    gh2 = (gh + 3.0 * rng.standard_normal(m)).astype(np.float32)
    F2, G2 = dev(fh2, gh2)
    check(fh2, gh2, F2, G2)
    assert prep.variant_state()["tiles_tested"] > before  # rows with keys: the launch was counted
    # arbitrary numbers in the key arrays
    kx.copy_(torch.from_numpy(rng.integers(-5, m + 5, n).astype(np.int32)))
    ky.copy_(torch.from_numpy(rng.integers(-2**31, 2**31 - 1, m).astype(np.int32)))
    check(fh2, gh2, F2, G2)


@pytest.mark.parametrize("n,m,d,eps", [(3000, 4100, 64, 0.01), (2500, 2300, 20, 0.05), (1200, 9000, 33, 0.02),
                                       (2600, 2200, 8, 0.05), (300, 260, 16, 0.1), (130, 700, 5, 0.2),
                                       (64, 257, 64, 0.05)])
def test_carried_margins_leave_every_step_unchanged(n, m, d, eps):
    """On prepared planes the kernel with the coarse tile test carries margins from launch to
    launch and, once the potentials move little, runs in a sparse form that visits only the
    tiles whose margin may have been used up.  Every step of a long sequence must equal the plain
    launch on the same inputs, and the oracle: while the potentials settle, when they are then
    disturbed a little (the sparse form stays, with many margins used up), a lot (back to the
    pipelined form), when the kept keys are overwritten with arbitrary numbers, and when eps
    changes (margins of another problem must not be used)."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    rng = np.random.default_rng(41)
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    a = np.full(n, 1.0 / n, np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    b /= b.sum()
    la, lb = np.log(a), np.log(b)
    fh = (-(x * x).sum(1)).astype(np.float32)
    gh = (-(y * y).sum(1)).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    worst = [0.0]

    def step(F_in, G_in, e, with_oracle=False):
        f1, g1 = _symmetric_step_raw(X, Y, F_in, G_in, LA, LB, e, coarse=True, prepared=prep, **kw)
        f0, g0 = _symmetric_step_raw(X, Y, F_in, G_in, LA, LB, e, coarse=False, **kw)
        err = max(rel_err(f1, f0.cpu().numpy()), rel_err(g1, g0.cpu().numpy()))
        worst[0] = max(worst[0], err)
        assert err < 2e-6, err
        if with_oracle:
            wf, wg = oracle.symmetric_step(x, y, F_in.cpu().numpy(), G_in.cpu().numpy(), la, lb, e,
                                           1.0, 0.5, 1.0, 1.0)
            assert rel_err(f1, wf) < RTOL and rel_err(g1, wg) < RTOL
        return f1, g1

    def skipped():
        return prep.variant_state()["tiles_skipped"]

    for it in range(30):  # settles: the sparse form takes over
        F, G = step(F, G, eps, with_oracle=it in (0, 29))
    s0, t0 = skipped(), prep.variant_state()["tiles_tested"]
    big = min(n, m) >= 1000  # (small problems may have no tile that can be skipped)
    assert s0 > 0 or not big
    F, G = step(F, G, eps)
    st = prep.variant_state()
    assert st["tiles_skipped"] > s0 or not big  # a settled step skips tiles
    # a disturbance of about 60 base-2 units: many margins are used up, the sparse form stays
    amp = 60.0 * eps * np.log(2.0)
    G2 = G + torch.from_numpy((amp * (2 * rng.random(m) - 1)).astype(np.float32)).cuda()
    F2 = F + torch.from_numpy((amp * (2 * rng.random(n) - 1)).astype(np.float32)).cuda()
    F, G = step(F2, G2, eps, with_oracle=True)
    for it in range(4):
        F, G = step(F, G, eps)
    # a large one: back to the pipelined form, then settling again
    G2 = G + torch.from_numpy((20.0 * rng.standard_normal(m)).astype(np.float32)).cuda()
    F2 = F + torch.from_numpy((20.0 * rng.standard_normal(n)).astype(np.float32)).cuda()
    F, G = step(F2, G2, eps, with_oracle=True)
    for it in range(16):
        F, G = step(F, G, eps)
    s1 = skipped()
    F, G = step(F, G, eps)
    assert skipped() > s1 or not big  # sparse again
    # arbitrary numbers in the key arrays: rows no longer start where their last maximum says
    prep.best_keys(0).copy_(torch.from_numpy(rng.integers(-5, m + 5, n).astype(np.int32)))
    prep.best_keys(1).copy_(torch.from_numpy(rng.integers(-2**31, 2**31 - 1, m).astype(np.int32)))
    F, G = step(F, G, eps, with_oracle=True)
    F, G = step(F, G, eps)
    # another eps on the same planes, and back
    for e in (2.0 * eps, 2.0 * eps, eps, eps, eps):
        F, G = step(F, G, e, with_oracle=(e != eps))
    print("largest difference to the plain launch", worst[0])


def test_carried_margins_with_one_sided_launches():
    """The alternating solver's half-updates are one-sided launches on shared prepared planes: the
    margins' state goes with the matrix that holds the query rows, so both directions settle into
    the sparse form, and every half-update equals the plain launch."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import flashsinkhorn_lse_fused
    rng = np.random.default_rng(42)
    n, m, d, eps = 2600, 3100, 48, 0.02
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    la = np.log(np.full(n, 1.0 / n, np.float32))
    lb = np.log(np.full(m, 1.0 / m, np.float32))
    X, Y, LA, LB = dev(x, y, la, lb)
    F = -(X * X).sum(1)
    G = -(Y * Y).sum(1)
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    for it in range(40):
        for q, k, lw, out in ((X, Y, LB, "f"), (Y, X, LA, "g")):
            pot = G if out == "f" else F
            got = flashsinkhorn_lse_fused(q, k, pot, lw, eps, allow_tf32=False, _prepared=prep, _coarse=True)
            want = flashsinkhorn_lse_fused(q, k, pot, lw, eps, allow_tf32=False)
            assert rel_err(got, want.cpu().numpy()) < 2e-6
            if out == "f":
                F = 0.5 * (F + got)  # damped, so that the sequence settles
            else:
                G = 0.5 * (G + got)
    st = prep.variant_state()
    assert st["tiles_skipped"] > 0


@pytest.mark.parametrize("variant", [True, None])
def test_solver_with_the_coarse_tile_test_equals_the_plain_solve(monkeypatch, variant):
    """Fixed-eps solves on large clouds run the kernel variant with the coarse tile test, forced
    or chosen on the device; the potentials are the plain solve's to rounding, for two clouds,
    for the self problem (one half-update per step) and for one cloud with two weight vectors."""
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    rng = np.random.default_rng(32)
    n, m, d = 16500, 16400, 8
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    a = rng.random(n).astype(np.float32) + 0.5
    b = rng.random(m).astype(np.float32) + 0.5
    X, Y, A, B = dev(x, y, a / a.sum(), b / b.sum())
    kw = dict(use_epsilon_scaling=False, eps=0.05, n_iters=26, allow_tf32=False,
              return_prelast=True)
    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    info = {}
    want = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
    assert info["coarse"] is False
    wu = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A, **kw)
    A2 = torch.flip(A, dims=[0]).contiguous()
    want2 = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A2, **kw)
    monkeypatch.setattr(solvers, "COARSE_TEST", variant)
    got = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
    assert info["coarse"] is False  # the default only switches on larger clouds
    monkeypatch.setattr(solvers, "_COARSE_MIN_ROWS", 16384)
    got = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
    assert info["coarse"] == ("auto" if variant is None else variant)
    state = info["prepared"].variant_state()
    assert state["tiles_tested"] > 0
    if variant is None:  # the third counted step decided
        assert state["decisions"] == 3
    for u, v in zip(got, want):
        assert rel_err(u, v.cpu().numpy()) < 2e-5
    # the self problem keeps its single half-update per step
    ws = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A, **kw)
    # these potentials are small differences of shifted potentials of size |x|^2
    scale = float((X * X).sum(dim=1).max())
    for u, v in zip(ws, wu):
        assert float((u - v).abs().max()) < 2e-6 * scale
    assert float((ws[0] - ws[1]).abs().max()) == 0.0
    # one cloud passed twice with two weight vectors is an ordinary two-sided problem
    got2 = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A2, **kw)
    for u, v in zip(got2, want2):
        assert float((u - v).abs().max()) < 2e-6 * scale
    # the alternating solver (both conventions, one of them unbalanced) takes the same variant
    akw = [dict(eps=0.05, n_iters=10, allow_tf32=False, reach=1.5),
           dict(eps=0.05, n_iters=10, allow_tf32=False, ott_convention=True)]
    alt = [solvers.sinkhorn_flashstyle_alternating(X, Y, A, B, **k) for k in akw]
    # the paired self problems of a debiased divergence too
    px, py = solvers.sinkhorn_flashstyle_symmetric_self_pair(X, A, Y, B, **kw)
    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    for k, got_alt in zip(akw, alt):
        for u, v in zip(got_alt, solvers.sinkhorn_flashstyle_alternating(X, Y, A, B, **k)):
            assert float((u - v).abs().max()) < 2e-6 * scale
    qx, qy = solvers.sinkhorn_flashstyle_symmetric_self_pair(X, A, Y, B, **kw)
    for u, v in zip(px + py, qx + qy):
        assert float((u - v).abs().max()) < 2e-6 * scale
    for u, v in zip(px, wu):
        assert float((u - v).abs().max()) < 2e-6 * scale


@pytest.mark.parametrize("variant", [True, None])
@pytest.mark.parametrize("d", [128, 100])
def test_solvers_with_the_coarse_tile_test_on_rows_of_65_to_128_columns(monkeypatch, variant, d):
    """``lse_coarse128_kernel``: the same test on wider rows (no carried margins), forced or
    chosen on the device, in the symmetric solver, the alternating solver (balanced in the other
    convention, and unbalanced) and the paired self problems; against the plain solves and, for
    the symmetric solve, the fp64 oracle."""
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    rng = np.random.default_rng(33 + d)
    n, m = 2300, 2700
    x, _ = _clustered(rng, n, d, spread=0.4)
    y, _ = _clustered(rng, m, d, spread=0.4)
    x, y = 0.3 * x, 0.3 * y
    a = rng.random(n).astype(np.float32) + 0.5
    b = rng.random(m).astype(np.float32) + 0.5
    a, b = a / a.sum(), b / b.sum()
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(use_epsilon_scaling=False, eps=0.05, n_iters=20, allow_tf32=False)
    akw = [dict(eps=0.05, n_iters=10, allow_tf32=False, reach=1.5),
           dict(eps=0.05, n_iters=10, allow_tf32=False, ott_convention=True)]
    monkeypatch.setattr(solvers, "_COARSE_MIN_ROWS_WIDE", 2048)

    def run(info):
        return (solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw),
                [solvers.sinkhorn_flashstyle_alternating(X, Y, A, B, **k) for k in akw],
                solvers.sinkhorn_flashstyle_symmetric_self_pair(X, A, Y, B, **kw))

    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    info0, info1 = {}, {}
    want = run(info0)
    assert info0["coarse"] is False
    monkeypatch.setattr(solvers, "COARSE_TEST", variant)
    got = run(info1)
    assert info1["coarse"] == ("auto" if variant is None else variant)
    assert info1["prepared"].variant_state()["tiles_tested"] > 0
    scale = float((X * X).sum(dim=1).max())
    for u, v in zip(got[0], want[0]):
        assert float((u - v).abs().max()) < 2e-6 * scale
    # (alternating half-updates feed on each other: where two kernels round a row's largest
    # logit differently they do so by the same amount in every iteration, x.y does not change,
    # and the difference of the solves grows with the iterations until the contraction holds
    # it; the wide kernel therefore sums its cross products apart from the large terms)
    for g_alt, w_alt in zip(got[1], want[1]):
        for u, v in zip(g_alt, w_alt):
            assert float((u - v).abs().max()) < 2e-6 * scale
    for u, v in zip(got[2][0] + got[2][1], want[2][0] + want[2][1]):
        assert float((u - v).abs().max()) < 2e-6 * scale
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, eps=0.05, n_iters=20, use_epsilon_scaling=False)[:2]
    assert rel_err(got[0][0], wf) < RTOL and rel_err(got[0][1], wg) < RTOL


@pytest.mark.parametrize("extra", [dict(), dict(reach=1.5), dict(reach_x=0.8, reach_y=2.0)])
def test_long_solves_with_carried_margins_equal_the_plain_solve(monkeypatch, extra):
    """Sixty fixed-eps iterations, balanced and unbalanced: most of them run in the sparse form of
    the kernel with the coarse tile test (tiles skipped on their carried margins), and the
    potentials are the plain solve's to rounding."""
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    rng = np.random.default_rng(43)
    n, m, d = 16500, 17000, 24
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    a = rng.random(n).astype(np.float32) + 0.5
    b = rng.random(m).astype(np.float32) + 0.5
    X, Y, A, B = dev(x, y, a / a.sum(), b / b.sum())
    kw = dict(use_epsilon_scaling=False, eps=0.05, n_iters=60, allow_tf32=False, **extra)
    monkeypatch.setattr(solvers, "_COARSE_MIN_ROWS", 16384)
    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    want = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, **kw)
    monkeypatch.setattr(solvers, "COARSE_TEST", None)
    info = {}
    got = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
    assert info["coarse"] == "auto"
    state = info["prepared"].variant_state()
    assert not state["plain_selected"] and state["tiles_skipped"] > 0.3 * state["tiles_tested"]
    for u, v in zip(got, want):
        assert rel_err(u, v.cpu().numpy()) < 2e-5


def test_variant_choice_on_the_device():
    """FS_FLAG_COARSE_AUTO: every step enqueues both kernel variants and a word next to the
    prepared planes says which runs.  Each row's running maximum starts from its logit at the key
    that held the row's maximum in the step before, so from the second step on a peaked plan ends
    most tiles at the coarse test, sorted rows or not, and the variant stays; with a flat plan
    (large eps) every tile matters and the third counted step switches to the plain kernel for
    good.  Either way the potentials equal those of the forced variants to rounding, and a second
    run takes the same path bit for bit."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_steps_raw
    rng = np.random.default_rng(35)
    n, m, d = 6000, 5200, 64
    x, lx = _clustered(rng, n, d)
    y, ly = _clustered(rng, m, d)
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    cases = {
        "sorted clusters": (x[np.argsort(lx, kind="stable")], y[np.argsort(ly, kind="stable")], 0.01, True),
        "unsorted cloud": (rng.standard_normal((n, d)).astype(np.float32),
                           rng.standard_normal((m, d)).astype(np.float32), 0.01, True),
        "flat plan": (rng.standard_normal((n, d)).astype(np.float32),
                      rng.standard_normal((m, d)).astype(np.float32), 100.0, False),
    }
    for name, (xs, ys, eps, stays) in cases.items():
        steps = [(eps, 1.0, 1.0, 1.0)] + [(eps, 0.5, 1.0, 1.0)] * 7
        fh = (-(xs * xs).sum(1)).astype(np.float32)
        gh = (-(ys * ys).sum(1)).astype(np.float32)
        X, Y, F, G, LA, LB = dev(xs, ys, fh, gh, np.log(a), np.log(b))
        runs = {}
        for coarse in ("auto", "auto", True, False):
            prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
            out = _symmetric_steps_raw(X, Y, F, G, LA, LB, steps, cost_scale=1.0, prepared=prep,
                                       allow_tf32=False, coarse=coarse)
            st = prep.variant_state()
            if coarse == "auto":
                # the first step has no keys to start from and is not counted; the third counted
                # step decides
                assert st["decisions"] == 3 and st["tiles_tested"] > 0, (name, st)
                share = st["tiles_ended"] / st["tiles_tested"]
                assert st["plain_selected"] == (not stays), (name, st)
                assert (share >= 0.4) == stays, (name, share)
                if "auto" in runs:  # same path, same bits
                    assert torch.equal(out[0], runs["auto"][0]) and torch.equal(out[1], runs["auto"][1])
            else:
                assert (st["tiles_tested"] > 0) == coarse
            runs[coarse] = out
        # eps = 100 turns fp32 rounding of the log-sum-exp (about 1e-7 of values of size 1) into
        # 1e-5 of potentials of size 1
        tol = 2e-6 if eps < 1.0 else 1e-4
        for k in (0, 1):
            ref = runs[False][k].cpu().numpy()
            assert rel_err(runs["auto"][k], ref) < tol and rel_err(runs[True][k], ref) < tol, name


def test_variant_follows_a_schedule_of_decreasing_eps(monkeypatch):
    """eps-scaling (the reference's default schedule) starts on a flat plan and ends on a peaked
    one.  With the variant left to the device the solve starts on the plain kernel
    (FS_FLAG_START_PLAIN), which counts the tiles whose exponentials it leaves out; once that
    share has grown by 4 % of all tiles over the first launch's, the next step runs the variant
    with the coarse tile test, whose keys and counts then start afresh.  The potentials equal the plain solve's to rounding, the same
    inputs take the same path twice, and the debiased loss (its self terms on schedules of
    their own) equals the plain one."""
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    from flash_sinkhorn_amd import SamplesLoss
    rng = np.random.default_rng(37)
    n, m, d = 26000, 24500, 16
    x, _ = _clustered(rng, n, d)
    y, _ = _clustered(rng, m, d)
    a = np.full(n, 1.0 / n, np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    b /= b.sum()
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(blur=0.05, scaling=0.5, allow_tf32=False)
    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    f0, g0 = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, **kw)
    monkeypatch.setattr(solvers, "COARSE_TEST", None)
    runs = []
    for _ in range(2):
        info = {}
        f1, g1 = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
        st = info["prepared"].variant_state()
        assert info["coarse"] == "auto"
        # the last steps ran the coarse variant, and it had its three launches with counts
        assert not st["plain_selected"] and st["decisions"] == 3, st
        runs.append((f1, g1))
    assert torch.equal(runs[0][0], runs[1][0]) and torch.equal(runs[0][1], runs[1][1])
    assert rel_err(f1, f0.cpu().numpy()) < 2e-6 and rel_err(g1, g0.cpu().numpy()) < 2e-6
    loss = SamplesLoss("sinkhorn", blur=0.05, debias=True, allow_tf32=False)
    v1 = float(loss(X, Y))
    monkeypatch.setattr(solvers, "COARSE_TEST", False)
    v0 = float(loss(X, Y))
    assert abs(v1 - v0) <= 1e-5 * abs(v0) + 1e-6


def test_graph_replays_equal_eager_solves(monkeypatch):
    """Small solves are captured into a HIP graph on their second call and replayed afterwards.
    Every call (eager, capturing, replaying) is compared with the launch-by-launch solve of the
    same inputs, bit for bit, with eager work and synchronisations between the calls and fresh
    input values each time; then the same through SamplesLoss(debias=True) with a backward pass
    (xy solve and the paired self solves, each with a graph of its own)."""
    from flash_sinkhorn_amd import SamplesLoss, _graphs
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    rng = np.random.default_rng(41)
    n, m, d = 700, 650, 5
    kw = dict(use_epsilon_scaling=False, eps=0.05, n_iters=12, allow_tf32=False, return_prelast=True)
    _graphs.clear()
    scratch = torch.zeros(1 << 16, device="cuda")
    for call in range(5):
        x, y, a, b = inputs(50 + call, n, m, d)
        X, Y, A, B = dev(x, y, a, b)
        monkeypatch.setattr(_graphs, "ENABLED", False)
        want = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, **kw)
        want_self = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A, reach=1.2, **kw)
        monkeypatch.setattr(_graphs, "ENABLED", True)
        got = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, **kw)
        scratch.add_(1.0).mul_(0.5)  # unrelated eager work between replays
        torch.cuda.synchronize()
        got_self = solvers.sinkhorn_flashstyle_symmetric(X, X, A, A, reach=1.2, **kw)
        for u, v in zip(got + got_self, want + want_self):
            assert torch.equal(u, v), call
    keys = [k[0] for k in _graphs._cache]
    assert keys.count("symmetric") == 2 and all(e.graph is not None for e in _graphs._cache.values())
    # through the public loss: value and gradient, replay after replay
    loss_fn = SamplesLoss("sinkhorn", blur=0.2, debias=True, use_epsilon_scaling=False, eps=0.04,
                          n_iters=10, allow_tf32=False)
    for call in range(4):
        x, y, _, _ = inputs(70 + call, n, n, d)
        outs = []
        for enabled in (False, True):
            monkeypatch.setattr(_graphs, "ENABLED", enabled)
            X = torch.from_numpy(x).cuda().requires_grad_(True)
            Y = torch.from_numpy(y).cuda()
            loss = loss_fn(X, Y)
            (gx,) = torch.autograd.grad(loss, X)
            torch.cuda.synchronize()
            outs.append((loss.detach(), gx))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1]), call
    assert any(k[0] == "self pair" for k in _graphs._cache)
    x, y, a, b = oracle_small = inputs(90, n, m, d)
    f, g, fp, gp = solvers.sinkhorn_flashstyle_symmetric(*dev(x, y, a, b), **kw)  # a replay
    wf, wg, wfp, wgp = oracle.sinkhorn_symmetric(x, y, a, b, use_epsilon_scaling=False, eps=0.05,
                                                 n_iters=12, return_prelast=True)
    assert rel_err(f, wf) < RTOL and rel_err(g, wg) < RTOL and rel_err(fp, wfp) < RTOL
