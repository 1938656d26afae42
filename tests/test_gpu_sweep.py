"""The one-sweep form of a two-sided log-sum-exp step (``lse_sweep_kernel``).

On prepared planes a symmetric step whose potentials moved little in the step before takes both
sides' sums from one sweep over the logits: row sums lane by lane, column sums over lanes, no
running maximum.  Whether a step may do so is decided on the device (by the merge of the step
before, from the range of that step's sums), and a step whose sums leave the range the form
is exact in is redone by the two-sided kernel within the same call.
Every step below is compared with the two-sided kernel on the SAME inputs (2e-6 of the largest
potential, the bar the other kernel variants are held to against the plain kernel; times eps
where eps > 1, since a potential is eps times a logarithm whose fp32 rounding does not shrink)
and with the fp64 oracle (1e-4).
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def _problem(seed, n, m, d, zero_weights=False):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((n, d)) / np.sqrt(d)).astype(np.float32)
    y = (rng.standard_normal((m, d)) / np.sqrt(d) + 0.2).astype(np.float32)
    a = (rng.random(n) + 0.5).astype(np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    if zero_weights:
        a[::7] = 0.0
        b[3::11] = 0.0
    return x, y, a / a.sum(), b / b.sum()


def _steps(x, y, a, b, eps_list, *, sweep, alpha=0.5, damp=(1.0, 1.0), cost_scale=1.0, disturb=None,
           check_oracle_at=()):
    """Runs the steps on one set of prepared planes with the one-sweep form allowed or not; every
    step is also run by the two-sided kernel on the same inputs (without prepared planes) and the
    largest difference is returned, with the list of steps before which the form was allowed."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels._common import log_weights
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    X, Y, A, B = dev(x, y, a, b)
    la, lb = log_weights(A).contiguous(), log_weights(B).contiguous()
    F = (-cost_scale * (X * X).sum(1)).contiguous()
    G = (-cost_scale * (Y * Y).sum(1)).contiguous()
    shift_x = (cost_scale * (X * X).sum(1)).contiguous()
    shift_y = (cost_scale * (Y * Y).sum(1)).contiguous()
    old = _lib.SWEEP
    worst, allowed, outs = 0.0, [], []
    state = {}
    try:
        _lib.SWEEP = sweep
        prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
        kw = dict(cost_scale=cost_scale, damping_f=damp[0], damping_g=damp[1], allow_tf32=False,
                  shift_x=shift_x if damp[0] < 1 else None, shift_y=shift_y if damp[1] < 1 else None)
        for i, eps in enumerate(eps_list):
            if disturb is not None and i in disturb:
                F = F + disturb[i][0]
                G = G + disturb[i][1]
            allowed.append(prep.variant_state()["sweep_next"])
            al = 1.0 if i == 0 else alpha
            f1, g1 = _symmetric_step_raw(X, Y, F, G, la, lb, eps, alpha=al, prepared=prep, **kw)
            _lib.SWEEP = False
            f0, g0 = _symmetric_step_raw(X, Y, F, G, la, lb, eps, alpha=al, **kw)
            _lib.SWEEP = sweep
            scale = max(float(f0.abs().max()), float(g0.abs().max()))
            err = max(float((f1 - f0).abs().max()), float((g1 - g0).abs().max())) / scale
            assert np.isfinite(err)
            worst = max(worst, err / max(1.0, eps))
            if i in check_oracle_at:
                wf, wg = oracle.symmetric_step(
                    x, y, F.cpu().numpy(), G.cpu().numpy(), oracle.log_weights(a), oracle.log_weights(b),
                    eps, cost_scale, al, damp[0], damp[1])
                for got, want in ((f1, wf), (g1, wg)):
                    e = np.abs(got.cpu().numpy().astype(np.float64) - want).max() / np.abs(want).max()
                    assert e < 1e-4, (i, e)
            outs.append((f1, g1))
            F, G = f1, g1
        state.update(prep.variant_state())
    finally:
        _lib.SWEEP = old
    return worst, allowed, _Outs(outs, state["sweep_redone"])


class _Outs(list):
    """The potentials of every step, and how many one-sweep steps the two-sided kernel redid."""

    def __init__(self, outs, redone):
        super().__init__(outs)
        self.redone = redone


@pytest.mark.parametrize("n,m,d", [(5000, 4700, 64), (2100, 9000, 32), (9100, 2300, 16),
                                   (4100, 4099, 5), (3000, 3300, 40), (3100, 2900, 128), (2048, 5100, 70)])
def test_one_sweep_steps_equal_two_sided_steps(n, m, d):
    x, y, a, b = _problem(n + d, n, m, d)
    worst, allowed, outs = _steps(x, y, a, b, [0.05] * 10, sweep=True, check_oracle_at=(5, 9))
    # the first step has nothing to go by; once the potentials move by less than a few base-2
    # units per step the form is allowed, and stays so
    assert not allowed[0] and allowed[-1] and sum(allowed) >= 5, allowed
    assert worst < 2e-6 and outs.redone == 0, (worst, outs.redone)
    # switched off, the state is never set
    worst0, allowed0, _ = _steps(x, y, a, b, [0.05] * 4, sweep=False)
    assert worst0 == 0.0 and not any(allowed0)


@pytest.mark.parametrize("n,m,d", [(2300, 2100, 200), (2048, 4500, 136), (3000, 2500, 520)])
def test_one_sweep_steps_at_more_than_128_columns(n, m, d):
    """The GEMM-style kernel's one-sweep form (``lse_gemm_kernel<3>``): the same permission, range
    check and fallback; key chunks whose last tile leaves a whole wavefront without keys."""
    x, y, a, b = _problem(n + d, n, m, d)
    worst, allowed, outs = _steps(x, y, a, b, [0.05] * 8, sweep=True, check_oracle_at=(4, 7))
    assert not allowed[0] and allowed[-1] and sum(allowed) >= 4, allowed
    assert worst < 2e-6 and outs.redone == 0, (worst, outs.redone)
    worst0, allowed0, _ = _steps(x, y, a, b, [0.05] * 3, sweep=False)
    assert worst0 == 0.0 and not any(allowed0)
    # bit for bit the same on a second run
    again = _steps(x, y, a, b, [0.05] * 8, sweep=True)[2]
    for (f0, g0), (f1, g1) in zip(outs, again):
        assert torch.equal(f0, f1) and torch.equal(g0, g1)


def test_a_jump_is_redone_at_more_than_128_columns():
    n, m, d = 2600, 2200, 256
    x, y, a, b = _problem(29, n, m, d)
    rng = np.random.default_rng(2)
    eps = 0.05
    jump = [t * 400.0 * eps for t in dev(rng.standard_normal(n).astype(np.float32),
                                         rng.standard_normal(m).astype(np.float32))]
    worst, allowed, outs = _steps(x, y, a, b, [eps] * 22, sweep=True, disturb={6: jump})
    assert allowed[6] and not allowed[7] and allowed[-1], allowed
    assert worst < 2e-6 and outs.redone == 1, (worst, outs.redone)


def _self_steps(x, y, a, b, eps_list, *, sweep, alpha=0.5, pair=True):
    """Steps of the self problems OT(x, x; a) and OT(y, y; b) on one set of prepared planes (the
    pair in one launch per step, or with ``pair=False`` the first one alone through the
    symmetric-step call); every step is also run by the two-sided kernel on the same inputs."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels._common import log_weights
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (_self_pair_steps_raw,
                                                                         _symmetric_step_raw)
    X, Y, A, B = dev(x, y, a, b)
    la, lb = log_weights(A).contiguous(), log_weights(B).contiguous()
    Fx, Fy = (-(X * X).sum(1)).contiguous(), (-(Y * Y).sum(1)).contiguous()
    old = _lib.SWEEP
    worst, allowed, outs = 0.0, [], []
    try:
        _lib.SWEEP = sweep
        fl = _lib.flags(True, False)
        prep = _lib.PreparedOperands(X, Y, fl, self_pair=True) if pair else _lib.PreparedOperands(X, X, fl)
        for i, eps in enumerate(eps_list):
            allowed.append(prep.variant_state()["sweep_next"])
            al = 1.0 if i == 0 else alpha
            if pair:
                run = lambda p: _self_pair_steps_raw(X, Y, Fx, Fy, la, lb, [(eps, eps, al, 1.0, 1.0)],
                                                     cost_scale=1.0, allow_tf32=False, prepared=p)
            else:
                run = lambda p: (_symmetric_step_raw(X, X, Fx, Fx, la, la, eps, cost_scale=1.0, alpha=al,
                                                     damping_f=1.0, damping_g=1.0, allow_tf32=False,
                                                     prepared=p)[0], Fy)
            f1x, f1y = run(prep)
            _lib.SWEEP = False
            f0x, f0y = run(None)
            _lib.SWEEP = sweep
            for got, want in ((f1x, f0x), (f1y, f0y)):
                err = float((got - want).abs().max()) / float(want.abs().max())
                assert np.isfinite(err)
                worst = max(worst, err / max(1.0, eps))
            if i == len(eps_list) - 1:
                for pts, F, lw, got in ((x, Fx, a, f1x),) + (((y, Fy, b, f1y),) if pair else ()):
                    lwo = oracle.log_weights(lw)
                    want = oracle.symmetric_step(pts, pts, F.cpu().numpy(), F.cpu().numpy(), lwo, lwo,
                                                 eps, 1.0, al, 1.0, 1.0)[0]
                    e = np.abs(got.cpu().numpy().astype(np.float64) - want).max() / np.abs(want).max()
                    assert e < 1e-4, e
            outs.append((f1x, f1y))
            Fx, Fy = f1x, f1y
        redone = prep.variant_state()["sweep_redone"]
    finally:
        _lib.SWEEP = old
    return worst, allowed, _Outs(outs, redone)


@pytest.mark.parametrize("n,m,d", [(4200, 3100, 32), (2048, 2500, 64), (5000, 6100, 16), (2300, 9000, 7),
                                   (2300, 2100, 200), (2048, 3900, 136), (2700, 3300, 128), (4500, 2100, 96)])
def test_self_problems_take_the_tiles_on_and_above_the_diagonal(n, m, d):
    """The two self problems of a debiased loss: the matrix of logits is symmetric once both
    biases are inside the exponent, and the one-sweep launch visits only the key tiles at or
    beyond a workgroup's own rows (row counts that are no multiple of the 256-row groups, a
    cloud of exactly 2048 rows, clouds of different sizes sharing the launch)."""
    x, y, a, b = _problem(n + m + d, n, m, d)
    worst, allowed, outs = _self_steps(x, y, a, b, [0.05] * 9, sweep=True)
    assert not allowed[0] and allowed[-1] and sum(allowed) >= 4, allowed
    assert worst < 2e-6 and outs.redone == 0, (worst, outs.redone)
    worst0, allowed0, _ = _self_steps(x, y, a, b, [0.05] * 3, sweep=False)
    assert worst0 == 0.0 and not any(allowed0)
    again = _self_steps(x, y, a, b, [0.05] * 9, sweep=True)[2]
    for (f0, g0), (f1, g1) in zip(outs, again):
        assert torch.equal(f0, f1) and torch.equal(g0, g1)


def test_a_single_self_problem_takes_the_form_too():
    x, y, a, b = _problem(31, 4700, 2100, 24)
    worst, allowed, outs = _self_steps(x, y, a, b, [0.1] * 8, sweep=True, pair=False)
    assert allowed[-1] and worst < 2e-6 and outs.redone == 0, (allowed, worst, outs.redone)


def test_one_sweep_steps_are_repeatable_bit_for_bit():
    x, y, a, b = _problem(5, 4400, 5200, 64)
    runs = [_steps(x, y, a, b, [0.1] * 8, sweep=True) for _ in range(2)]
    assert runs[0][1] == runs[1][1] and runs[0][1][-1]
    for (f0, g0), (f1, g1) in zip(runs[0][2], runs[1][2]):
        assert torch.equal(f0, f1) and torch.equal(g0, g1)


def test_unbalanced_steps_take_the_one_sweep_form_too():
    """Damped updates (reach) and their shift correction live in the epilogue, which both merges share."""
    x, y, a, b = _problem(11, 3900, 4300, 32)
    worst, allowed, _ = _steps(x, y, a, b, [0.1] * 10, sweep=True, damp=(0.8, 0.6), cost_scale=0.5)
    assert allowed[-1] and worst < 2e-6, (allowed, worst)


def test_empty_weights_keep_the_two_sided_kernel():
    """A row or key of weight zero has no mass in the plan: its sum is 0 in the one-sweep form,
    which therefore never gets the permission; the results are the two-sided kernel's."""
    x, y, a, b = _problem(13, 3000, 2600, 16, zero_weights=True)
    worst, allowed, _ = _steps(x, y, a, b, [0.1] * 6, sweep=True)
    assert not any(allowed) and worst == 0.0, (allowed, worst)


def test_a_jump_of_the_potentials_is_redone_by_the_two_sided_kernel():
    """With the form allowed, potentials that suddenly move by hundreds of base-2 units push the
    sums out of the range the form is exact in (or to infinity): the merge notices, the two-sided
    kernel redoes the step inside the same call (bit-equal to a two-sided step), and the form
    stays off until a step has settled again."""
    n, m, d = 4000, 3600, 64
    x, y, a, b = _problem(17, n, m, d)
    rng = np.random.default_rng(1)
    eps = 0.05
    jump = [t * 400.0 * eps for t in dev(rng.standard_normal(n).astype(np.float32),
                                         rng.standard_normal(m).astype(np.float32))]
    worst, allowed, outs = _steps(x, y, a, b, [eps] * 22, sweep=True, disturb={6: jump})
    assert allowed[6] and not allowed[7] and allowed[-1], allowed
    assert worst < 2e-6 and outs.redone == 1, (worst, outs.redone)
    # the step with the jump, alone: the same numbers as the two-sided kernel, bit for bit
    _, allowed2, outs2 = _steps(x, y, a, b, [eps] * 7, sweep=True, disturb={6: jump})
    _, _, outs0 = _steps(x, y, a, b, [eps] * 7, sweep=False, disturb={6: jump})
    # (up to step 5 the two runs differ by rounding, so only the mechanism is compared here:
    # step 6 of the first run was checked against the two-sided kernel on its own inputs above)
    assert allowed2[6] and len(outs2) == len(outs0)


def test_a_schedule_of_decreasing_eps_keeps_the_form_while_the_plan_is_flat():
    """The permission goes by the sums of the step before, not by eps: while the sums stay in
    range when eps is halved (on a flat plan they hardly move) the steps of a schedule take the
    form one after the other; a step whose sums leave the range would be redone.  Every step
    equals the two-sided kernel's on the same inputs whichever way it went."""
    x, y, a, b = _problem(19, 3500, 3700, 32)
    eps_list = [64.0 * 0.5 ** k for k in range(14)]  # 64 ... 0.008
    worst, allowed, outs = _steps(x, y, a, b, eps_list, sweep=True, check_oracle_at=(4, 13))
    assert allowed[1] and allowed[4], allowed
    assert worst < 2e-6 and outs.redone <= 2, (worst, outs.redone)
    # the same on clouds nine times as far apart (in cost), where the plan peaks earlier
    worst, allowed, outs = _steps(3.0 * x, 3.0 * y, a, b, eps_list, sweep=True, check_oracle_at=(13,))
    assert allowed[1] and worst < 2e-6 and outs.redone <= 2, (allowed, worst, outs.redone)


def test_solver_results_do_not_depend_on_the_form(monkeypatch):
    """A fixed-eps solve (plain kernel variant) with the form allowed and not: the same
    potentials to rounding, and equal to the fp64 oracle's solve."""
    import flash_sinkhorn_amd.sinkhorn_solvers as solvers
    from flash_sinkhorn_amd import _graphs, _lib
    monkeypatch.setattr(_graphs, "ENABLED", False)  # (a replayed run keeps its planes to itself)
    x, y, a, b = _problem(23, 2600, 2900, 8)
    X, Y, A, B = dev(x, y, a, b)
    kw = dict(use_epsilon_scaling=False, eps=0.1, n_iters=30, allow_tf32=False)
    monkeypatch.setattr(_lib, "SWEEP", False)
    f0, g0 = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, **kw)
    monkeypatch.setattr(_lib, "SWEEP", True)
    info = {}
    f1, g1 = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, solve_info=info, **kw)
    assert info["prepared"].variant_state()["sweep_next"]
    scale = float(f0.abs().max())
    assert float((f1 - f0).abs().max()) < 1e-5 * scale and float((g1 - g0).abs().max()) < 1e-5 * scale
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, eps=0.1, n_iters=30, use_epsilon_scaling=False)[:2]
    for got, want in ((f1, wf), (g1, wg)):
        assert np.abs(got.cpu().numpy() - want).max() / np.abs(want).max() < 1e-4


@pytest.mark.parametrize("seed", range(4))
def test_random_shapes_take_the_form_without_changing_results(seed):
    """Seeded random shapes on both sides of each kernel family's width limits (64, 128), row
    counts from one workgroup's worth down to a single row, zero weights now and then: steps of
    xy pairs, of the pair of self problems and of a single one.  eps stays below 0.3: at large eps
    a self problem's potentials nearly cancel against |x|^2, and an error measured against the
    largest potential says little."""
    rng = np.random.default_rng(4000 + seed)
    widths = [1, 3, 16, 17, 33, 63, 64, 65, 70, 96, 127, 128, 129, 136, 200, 257, 300]
    for case in range(14):
        d = int(rng.choice(widths))
        n, m = int(rng.integers(1, 2600)), int(rng.integers(1, 2600))
        eps = float(10 ** rng.uniform(-1.7, -0.55))
        steps = int(rng.integers(3, 8))
        kind = int(rng.integers(0, 3))  # xy pair, pair of self problems, one self problem
        x, y, a, b = _problem(int(rng.integers(0, 1 << 30)), n, m, d, zero_weights=bool(rng.random() < 0.3))
        if kind == 0:
            worst, allowed, outs = _steps(x, y, a, b, [eps] * steps, sweep=True)
        else:
            worst, allowed, outs = _self_steps(x, y, a, b, [eps] * steps, sweep=True, pair=(kind == 1))
        assert worst < 2e-6, (seed, case, n, m, d, eps, steps, kind, worst)
