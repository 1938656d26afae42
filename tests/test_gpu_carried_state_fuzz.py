"""Seeded random walks over the state that ``lse_coarse_kernel`` carries from launch to launch.

On prepared planes the kernel keeps, per row, the key of the row's largest logit, that logit,
the key biases of the last launch and, per 32-row block and 32-key sub-tile, a margin with a
generation tag; state words say which form of the kernel runs.  Whatever sequence of launches
touches that state, every launch must return what the plain kernel returns on the same inputs.
The walks below mix, in random order: Jacobi steps that let the potentials settle, small and
large disturbances of the potentials, changes of eps (each starts a new generation of margins:
the long walk passes the 255 generations an entry can name), the two clouds swapping roles,
key arrays overwritten with arbitrary numbers, and one-sided launches in either direction.
Every step is held to 2e-6 (max norm, relative to the largest potential) against the plain
launch, which the other tests hold to 1e-4 against the fp64 oracle; the walk stops at the first
step that fails and names it.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _clouds(rng, n, m, d):
    centres = rng.standard_normal((6, d)) * 2.0
    x = (centres[rng.integers(0, 6, n)] + rng.standard_normal((n, d))).astype(np.float32)
    y = (centres[rng.integers(0, 6, m)] + rng.standard_normal((m, d))).astype(np.float32)
    return x, y


def _walk(seed, n, m, d, eps0, steps, p_eps):
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        _symmetric_step_raw, flashsinkhorn_lse_fused)
    rng = np.random.default_rng(seed)
    x, y = _clouds(rng, n, m, d)
    X, Y = torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()
    b = (rng.random(m) + 0.5).astype(np.float32)
    LA = torch.full((n,), -float(np.log(n)), device="cuda")
    LB = torch.from_numpy(np.log(b / b.sum())).cuda()
    F, G = -(X * X).sum(1), -(Y * Y).sum(1)
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    eps = eps0
    swapped = False
    worst = 0.0
    counts = {}

    def noise(k, amp):
        return torch.from_numpy((amp * rng.standard_normal(k)).astype(np.float32)).cuda()

    for it in range(steps):
        u = rng.random()
        if u < p_eps:
            act = "eps"
            eps = eps0 * float(rng.choice([1.0, 1.5, 2.0, 0.75]))
        elif u < p_eps + 0.08:
            act = "small disturbance"  # a few base-2 units: margins are used up one by one
            amp = float(rng.uniform(1.0, 40.0)) * eps * np.log(2.0)
            F, G = F + noise(n, amp), G + noise(m, amp)
        elif u < p_eps + 0.12:
            act = "large disturbance"  # far past any margin
            F, G = F + noise(n, 10.0), G + noise(m, 10.0)
        elif u < p_eps + 0.17:
            act = "swap roles"
            swapped = not swapped
        elif u < p_eps + 0.21:
            act = "overwrite keys"
            prep.best_keys(0).copy_(torch.from_numpy(rng.integers(-5, m + 5, n).astype(np.int32)))
            prep.best_keys(1).copy_(torch.from_numpy(
                rng.integers(-2**31, 2**31 - 1, m).astype(np.int32)))
        elif u < p_eps + 0.33:
            act = "one-sided f" if rng.random() < 0.5 else "one-sided g"
        else:
            act = "step"
        counts[act] = counts.get(act, 0) + 1
        if act.startswith("one-sided"):
            q, k, pot, lw = (X, Y, G, LB) if act.endswith("f") else (Y, X, F, LA)
            got = flashsinkhorn_lse_fused(q, k, pot, lw, eps, allow_tf32=False, _prepared=prep,
                                          _coarse=True)
            want = flashsinkhorn_lse_fused(q, k, pot, lw, eps, allow_tf32=False)
            err = float((got - want).abs().max() / want.abs().max())
            if act.endswith("f"):
                F = 0.5 * (F + got)
            else:
                G = 0.5 * (G + got)
        else:
            args = (Y, X, G, F, LB, LA) if swapped else (X, Y, F, G, LA, LB)
            o1, o2 = _symmetric_step_raw(*args, eps, coarse=True, prepared=prep, **kw)
            p1, p2 = _symmetric_step_raw(*args, eps, coarse=False, **kw)
            scale = max(float(p1.abs().max()), float(p2.abs().max()))
            err = max(float((o1 - p1).abs().max()), float((o2 - p2).abs().max())) / scale
            F, G = (o2, o1) if swapped else (o1, o2)
        worst = max(worst, err)
        assert err < 2e-6, (f"seed {seed}, shape {n} x {m} x {d}, step {it} ({act}, eps {eps:g}, "
                            f"roles swapped: {swapped}): differs from the plain launch by {err:.3e}")
    state = prep.variant_state()
    print(f"walk seed {seed} {n}x{m}x{d}: {steps} steps {counts}, largest difference to the plain "
          f"launch {worst:.2e}, units not visited {state['tiles_skipped']}, tested "
          f"{state['tiles_tested']}")
    return state


@pytest.mark.parametrize("seed,n,m,d,eps", [(1, 2600, 2200, 32, 0.02), (2, 1500, 3100, 64, 0.01),
                                            (3, 3000, 2900, 16, 0.05), (4, 700, 4200, 8, 0.05)])
def test_random_walks_over_the_carried_state(seed, n, m, d, eps):
    state = _walk(seed, n, m, d, eps, steps=160, p_eps=0.04)
    assert state["tiles_skipped"] > 0  # the sparse form ran, with margins that held


def test_random_walk_past_255_generations_of_margins():
    """An entry names its generation in 8 bits; after 255 generations on one set of planes the
    margins of that role must stay off rather than match a stale entry."""
    _walk(5, 1300, 1100, 32, 0.02, steps=640, p_eps=0.7)
