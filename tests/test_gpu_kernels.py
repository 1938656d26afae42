"""HIP kernels (through the C ABI) vs the fp64 oracle on seeded inputs.

Tolerance: north-star bar is rel 1e-4 on potentials and gradients for fp32;
errors are measured relative to the largest magnitude of the expected output.
"""
import numpy as np
import pytest
import torch

import oracle
from tests.golden.recipe import inputs

pytestmark = pytest.mark.gpu
RTOL = 1e-4

SHAPES = [  # (n, m, d): ragged tiles, d not a multiple of 4/8, every padded width
    (64, 48, 32), (300, 257, 64), (129, 1000, 3), (1000, 130, 20), (257, 300, 128),
    (70, 65, 100), (4500, 3000, 64), (33, 5, 8), (1, 1, 1),
    # two row blocks per wavefront at the narrow widths (2048 rows and more)
    (2100, 2300, 20), (2050, 300, 3),
    # column-sliced kernels (d > 128): every (wavefronts, slice) configuration, ragged d
    (100, 90, 200), (64, 70, 512), (50, 140, 700), (40, 33, 1536), (33, 20, 1030), (70, 300, 130),
    (600, 2000, 256),
    # wider than one workgroup's 1536 columns: super-slices
    (40, 50, 2048), (33, 70, 3100),
    # GEMM-shaped large-d kernels: several key tiles, ragged key splits, column groups + splits
    (64, 2048, 160), (100, 1100, 300), (40, 600, 2048),
]


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def rel_err(got, want):
    got = got.detach().cpu().numpy().astype(np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def problem(n, m, d, seed=0, eps=0.3):
    x, y, a, b = inputs(100 + seed, n, m, d, scale=1.0 / np.sqrt(max(d, 1)) * 2.0)
    rng = np.random.default_rng(seed + 7)
    f_hat = rng.standard_normal(n).astype(np.float32) * 0.3
    g_hat = rng.standard_normal(m).astype(np.float32) * 0.3
    return x, y, a, b, f_hat, g_hat


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_lse_raw_and_fused(n, m, d):
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_lse, flashsinkhorn_lse_fused)
    x, y, a, b, f_hat, g_hat = problem(n, m, d)
    eps = 0.3
    lb = np.log(b)
    bias = (g_hat / eps + lb).astype(np.float32)
    X, Y, B, G, LB = dev(x, y, bias, g_hat, lb)
    for cs, damp in ((1.0, 1.0), (0.5, 0.7)):
        want = oracle.lse_shifted(x, y, bias, eps, cs, damp)
        got = flashsinkhorn_lse(X, Y, B, eps, cost_scale=cs, damping=damp, allow_tf32=False)
        assert rel_err(got, want) < RTOL
        want = oracle.lse_shifted_fused(x, y, g_hat, lb, eps, cs, damp)
        got = flashsinkhorn_lse_fused(X, Y, G, LB, eps, cost_scale=cs, damping=damp,
                                      allow_tf32=False)
        assert rel_err(got, want) < RTOL


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_symmetric_step(n, m, d):
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_symmetric_step)
    x, y, a, b, f_hat, g_hat = problem(n, m, d, seed=1)
    la, lb = np.log(a), np.log(b)
    X, Y, F, G, LA, LB = dev(x, y, f_hat, g_hat, la, lb)
    for alpha, df, dg in ((0.5, 1.0, 1.0), (1.0, 0.8, 0.6)):
        wf, wg = oracle.symmetric_step(x, y, f_hat, g_hat, la, lb, 0.25, 0.5, alpha, df, dg)
        gf, gg = flashsinkhorn_symmetric_step(X, Y, F, G, LA, LB, 0.25, cost_scale=0.5,
                                              alpha=alpha, damping_f=df, damping_g=dg,
                                              allow_tf32=False)
        assert rel_err(gf, wf) < RTOL and rel_err(gg, wg) < RTOL


def test_lse_small_eps_large_logits():
    # eps = 0.01 with |x.y| ~ 50: logits of order 1e4, the regime of the headline config
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import flashsinkhorn_lse_fused
    x, y, a, b = inputs(5, 700, 900, 64, y_shift=0.5)
    be = (y.astype(np.float64) ** 2).sum(1)
    g_hat = (-be).astype(np.float32)
    lb = np.log(b)
    want = oracle.lse_shifted_fused(x, y, g_hat, lb, 0.01)
    got = flashsinkhorn_lse_fused(*dev(x, y, g_hat, lb), 0.01, allow_tf32=False)
    assert rel_err(got, want) < RTOL


def test_zero_weight_and_masked_bias():
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_lse, flashsinkhorn_lse_fused)
    from flash_sinkhorn_amd.kernels._common import log_weights
    x, y, a, b, f_hat, g_hat = problem(90, 70, 16)
    b = b.copy(); b[::3] = 0.0
    LB = log_weights(torch.from_numpy(b).cuda())
    want = oracle.lse_shifted_fused(x, y, g_hat, oracle.log_weights(b), 0.3)
    got = flashsinkhorn_lse_fused(*dev(x, y, g_hat), LB, 0.3, allow_tf32=False)
    assert rel_err(got, want) < RTOL
    bias = (g_hat / 0.3).astype(np.float32); bias[5:] = -np.inf  # only 5 live keys
    want = oracle.lse_shifted(x, y, bias, 0.3)
    got = flashsinkhorn_lse(*dev(x, y, bias), 0.3, allow_tf32=False)
    assert rel_err(got, want) < RTOL


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_gradient(n, m, d):
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    x, y, a, b, f, g = problem(n, m, d, seed=2)
    gs = np.array([0.7], np.float32)
    wx, wy = oracle.grad_barycentric(x, y, a, b, f, g, 0.3, cost_scale=0.5, grad_scale=0.7)
    X, Y, A, B, F, G, GS = dev(x, y, a, b, f, g, gs)
    gx, gy = grad(X, Y, A, B, F, G, eps=0.3, cost_scale=0.5, grad_scale=GS, allow_tf32=False)
    assert rel_err(gx, wx) < RTOL and rel_err(gy, wy) < RTOL
    gx, gy = grad(X, Y, A, B, F, G, eps=0.3, cost_scale=0.5, grad_scale=GS, allow_tf32=False,
                  compute_grad_y=False)
    assert gy is None and rel_err(gx, wx) < RTOL
    gx, gy = grad(X, Y, A, B, F, G, eps=0.3, cost_scale=0.5, grad_scale=GS, allow_tf32=False,
                  compute_grad_x=False)
    assert gx is None and rel_err(gy, wy) < RTOL


@pytest.mark.parametrize("n,m,d,eps", [(3000, 4100, 64, 0.01), (2100, 2300, 20, 0.05), (700, 5000, 100, 0.02),
                                       (129, 1000, 3, 0.05)])
def test_gradient_on_peaked_plans_with_and_without_key_hints(n, m, d, eps):
    """The product kernel leaves out 32 x 32 tiles whose logits all lie 2^40 below the rows'
    running maxima, and starts those maxima from the rows' logits at keys a caller names
    (fs_grad_seeded).  On a peaked plan (clustered clouds, small eps) the gradient must equal the
    fp64 oracle with the arg-max keys, with keys of another problem, with arbitrary numbers and
    without keys, and the hinted and plain results must agree to rounding."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(51)
    # (norms of order 1: the standard potentials enter the logits as g / eps, and their fp32
    # rounding must stay far below one logit unit for the comparison to be about the kernel)
    sc = 0.7 / np.sqrt(d)
    centres = rng.standard_normal((8, d)) * 2.0
    x = (sc * (centres[rng.integers(0, 8, n)] + rng.standard_normal((n, d)))).astype(np.float32)
    y = (sc * (centres[rng.integers(0, 8, m)] + rng.standard_normal((m, d)))).astype(np.float32)
    a = np.full(n, 1.0 / n, np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    b /= b.sum()
    # potentials of a few symmetric iterations: a peaked plan, not a converged one
    fh = -(x * x).sum(1).astype(np.float32)
    gh = -(y * y).sum(1).astype(np.float32)
    la, lb = np.log(a), np.log(b)
    for it in range(4):
        fh, gh = oracle.symmetric_step(x, y, fh, gh, la, lb, eps, 1.0, 1.0 if it == 0 else 0.5, 1.0, 1.0)
    f = (fh + (x * x).sum(1)).astype(np.float32)
    g = (gh + (y * y).sum(1)).astype(np.float32)
    wx, wy = oracle.grad_barycentric(x, y, a, b, f, g, eps, cost_scale=1.0, grad_scale=1.0)
    logits = (2.0 * x.astype(np.float64) @ y.astype(np.float64).T + gh[None, :]) / eps + lb[None, :]
    kx_true = logits.argmax(1).astype(np.int32)
    logits_t = (2.0 * y.astype(np.float64) @ x.astype(np.float64).T + fh[None, :]) / eps + la[None, :]
    ky_true = logits_t.argmax(1).astype(np.int32)
    X, Y, A, B, F, G = dev(x, y, a, b, f, g)
    plain = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False)
    assert rel_err(plain[0], wx) < RTOL and rel_err(plain[1], wy) < RTOL
    hints = [(kx_true, ky_true),
             (rng.integers(0, m, n).astype(np.int32), rng.integers(0, n, m).astype(np.int32)),
             (rng.integers(-2**31, 2**31 - 1, n).astype(np.int32), np.full(m, -1, np.int32))]
    for kx, ky in hints:
        keys = (torch.from_numpy(kx).cuda(), torch.from_numpy(ky).cuda())
        gx, gy = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, _seed_keys=keys)
        assert rel_err(gx, wx) < RTOL and rel_err(gy, wy) < RTOL
        assert rel_err(gx, plain[0].cpu().numpy()) < RTOL and rel_err(gy, plain[1].cpu().numpy()) < RTOL
    gx, _ = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, compute_grad_y=False,
                 _seed_keys=(torch.from_numpy(kx_true).cuda(), torch.from_numpy(ky_true).cuda()))
    assert rel_err(gx, wx) < RTOL


@pytest.mark.parametrize("d", [100, 128, 72])
def test_key_hints_on_rows_wider_than_64_columns(d):
    """64 < d <= 128: the logit at a hinted key must be the dot product over ALL columns.  Every
    row is hinted at a key whose first 64 columns repeat the row (large positive half dot) and
    whose other columns oppose it (large negative half dot): the whole logit lies far below the
    64-column part, and a starting value taken from that part alone would sit above every logit
    of the row, so that each tile is left out.  Hinted, unhinted and the fp64 oracle must agree."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(61)
    n = m = 640
    eps = 0.02
    x = rng.standard_normal((n, d))
    x[:, :64] *= 1.6 / np.linalg.norm(x[:, :64], axis=1, keepdims=True)
    x[:, 64:] *= 0.6 / np.linalg.norm(x[:, 64:], axis=1, keepdims=True)
    x = x.astype(np.float32)
    y = np.concatenate([x[:, :64], -3.0 * x[:, 64:]], axis=1)
    y = (y + 0.01 * rng.standard_normal((m, d))).astype(np.float32)
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    la, lb = np.log(a), np.log(b)
    # potentials that take the key norms out of the logits: what is left is 2 x.y / eps
    f = (0.02 * rng.standard_normal(n)).astype(np.float32)
    g = ((y.astype(np.float64) ** 2).sum(1) + 0.02 * rng.standard_normal(m)).astype(np.float32)
    gh = g - (y.astype(np.float64) ** 2).sum(1)
    # the half dot of the hinted key exceeds every whole logit of its row by more than 2^40
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    logits = (2.0 * x64 @ y64.T + gh[None, :]) / eps + lb[None, :]
    half = (2.0 * (x64[:, :64] * y64[:, :64]).sum(1) + gh) / eps + lb
    assert ((half - logits.max(1)) * np.log2(np.e)).min() > 40.0
    wx, wy = oracle.grad_barycentric(x, y, a, b, f, g, eps)
    X, Y, A, B, F, G = dev(x, y, a, b, f, g)
    plain = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False)
    own = torch.arange(n, dtype=torch.int32, device="cuda")
    gx, gy = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, _seed_keys=(own, own))
    assert rel_err(gx, wx) < RTOL and rel_err(gy, wy) < RTOL
    assert rel_err(gx, plain[0].cpu().numpy()) < RTOL and rel_err(gy, plain[1].cpu().numpy()) < RTOL


def test_key_hints_that_name_masked_keys():
    """Hints may name keys that are masked out (potential -inf: bias at the finite stand-in for
    -inf) or that carry no weight (log-weight floor -100000): such a key says nothing about its
    row's largest logit, and the result must not depend on it."""
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(62)
    n, m, d, eps = 700, 900, 64, 0.02
    sc = 0.7 / np.sqrt(d)
    centres = rng.standard_normal((6, d)) * 2.0
    x = (sc * (centres[rng.integers(0, 6, n)] + rng.standard_normal((n, d)))).astype(np.float32)
    y = (sc * (centres[rng.integers(0, 6, m)] + rng.standard_normal((m, d)))).astype(np.float32)
    a = np.full(n, 1.0 / n, np.float32)
    b = (rng.random(m) + 0.5).astype(np.float32)
    dead = rng.choice(m, 40, replace=False)
    b[dead[:20]] = 0.0                      # no weight
    b /= b.sum()
    f = (0.1 * rng.standard_normal(n)).astype(np.float32)
    g = (0.1 * rng.standard_normal(m)).astype(np.float32)
    g[dead[20:]] = -np.inf                  # masked by the potential
    wx, _ = oracle.grad_barycentric(x, y, a, b, f, g, eps)
    X, Y, A, B, F, G = dev(x, y, a, b, f, g)
    plain, _ = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, compute_grad_y=False)
    assert rel_err(plain, wx) < RTOL
    kx = rng.integers(0, m, n).astype(np.int32)
    kx[::2] = dead[rng.integers(0, 40, len(kx[::2]))]   # every other row is hinted at a dead key
    keys = (torch.from_numpy(kx).cuda(), torch.zeros(m, dtype=torch.int32, device="cuda"))
    gx, _ = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, compute_grad_y=False, _seed_keys=keys)
    assert torch.isfinite(gx).all()
    assert rel_err(gx, wx) < RTOL and rel_err(gx, plain.cpu().numpy()) < RTOL


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_apply_vec_and_mat(n, m, d):
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    x, y, a, b, f_hat, g_hat = problem(n, m, d, seed=3)
    la, lb = np.log(a), np.log(b)
    rng = np.random.default_rng(4)
    vm, vn = rng.standard_normal(m).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    Vm = rng.standard_normal((m, d)).astype(np.float32)
    Vn = rng.standard_normal((n, d)).astype(np.float32)
    sc = rng.random(m).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, f_hat, g_hat, la, lb)
    kw = dict(eps=0.4, cost_scale=0.5)
    okw = dict(eps=0.4, cost_scale=0.5)
    got = apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, dev(vm)[0], axis=1, **kw)
    assert rel_err(got, oracle.apply_plan_vec(x, y, f_hat, g_hat, la, lb, vm, axis=1, **okw)) < RTOL
    got = apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, dev(vn)[0], axis=0, **kw)
    assert rel_err(got, oracle.apply_plan_vec(x, y, f_hat, g_hat, la, lb, vn, axis=0, **okw)) < RTOL
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, dev(Vm)[0], axis=1, scale=dev(sc)[0], **kw)
    want = oracle.apply_plan_mat(x, y, f_hat, g_hat, la, lb, Vm, axis=1, scale=sc, **okw)
    assert rel_err(got, want) < RTOL
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, Y, axis=1, **kw)  # values = key rows
    assert rel_err(got, oracle.apply_plan_mat(x, y, f_hat, g_hat, la, lb, y, axis=1, **okw)) < RTOL
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, dev(Vn)[0], axis=0, **kw)
    assert rel_err(got, oracle.apply_plan_mat(x, y, f_hat, g_hat, la, lb, Vn, axis=0, **okw)) < RTOL


@pytest.mark.parametrize("n,m,d", SHAPES)
def test_mat5(n, m, d):
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    x, y, a, b, f, g = problem(n, m, d, seed=5)
    A = np.random.default_rng(6).standard_normal((n, d)).astype(np.float32)
    f = f - 2.0  # keep exp((f+g-C)/eps) in a tame range
    want = oracle.mat5(x, y, f, g, A, 0.5, 0.5)
    got = mat5_sqeuclid(*dev(x, y, f, g, A), eps=0.5, cost_scale=0.5)
    assert rel_err(got, want) < RTOL


@pytest.mark.parametrize("n,m,d", [(17000, 3000, 64), (16500, 2500, 40), (16400, 700, 20)])
def test_products_with_two_row_blocks_per_wave(n, m, d):
    """From 16384 query rows on, the d <= 64 product kernels give every wavefront two blocks of
    32 rows (at 64 columns the matrix product then streams its key operands from LDS): sampled
    rows of plan*matrix, plan*vector, the gradient and the c-transform against the oracle."""
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    from flash_sinkhorn_amd import c_transform_fwd
    x, y, a, b, fh, gh = problem(n, m, d, seed=9)
    la, lb = np.log(a), np.log(b)
    rng = np.random.default_rng(10)
    V = rng.standard_normal((m, d)).astype(np.float32)
    v = rng.standard_normal(m).astype(np.float32)
    rows = np.concatenate([rng.choice(n, 120, replace=False), [0, 31, 32, 63, 64, n - 1]])
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    kw = dict(eps=0.4, cost_scale=0.5)
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, dev(V)[0], axis=1, allow_tf32=False, **kw)
    want = oracle.apply_plan_mat(x[rows], y, fh[rows], gh, la[rows], lb, V, axis=1, **kw)
    assert rel_err(got[torch.from_numpy(rows).cuda()], want) < RTOL
    got = apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, dev(v)[0], axis=1, allow_tf32=False, **kw)
    want = oracle.apply_plan_vec(x[rows], y, fh[rows], gh, la[rows], lb, v, axis=1, **kw)
    assert rel_err(got[torch.from_numpy(rows).cuda()], want) < RTOL
    gx, _ = grad(X, Y, *dev(a, b), F, G, eps=0.3, cost_scale=0.5, allow_tf32=False,
                 compute_grad_y=False)
    wx, _ = oracle.grad_barycentric(x[rows], y, a[rows], b, fh[rows], gh, 0.3, cost_scale=0.5)
    assert rel_err(gx[torch.from_numpy(rows).cuda()], wx) < RTOL
    psi = rng.standard_normal(m).astype(np.float32)
    c, _ = c_transform_fwd(X, Y, dev(psi)[0], cost_scale=0.5, allow_tf32=False)
    wc, _ = oracle.c_transform(x[rows], y, psi, 0.5)
    assert np.abs(c.cpu().numpy()[rows] - wc).max() <= 1e-5 * max(np.abs(wc).max(), 1.0)


@pytest.mark.parametrize("n,m,d,eps", [(40000, 200000, 4, 0.5), (30000, 120000, 16, 0.05)])
def test_long_key_chunks_keep_fp32_accuracy(n, m, d, eps):
    """Hundreds of key tiles per workgroup: whatever is applied once per tile (the rescale of
    the running sum, the offset of the exponents) must not carry a rounding residual, or the
    residuals add up.  Sampled rows against the fp64 oracle, 3e-6 of the largest potential
    (a residual of half an ulp of the running maximum per tile gives 2e-5 here)."""
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import flashsinkhorn_lse_fused
    rng = np.random.default_rng(17)
    x = rng.standard_normal((n, d)).astype(np.float32)
    y = (rng.standard_normal((m, d)) + 0.3).astype(np.float32)
    gh = (-(y * y).sum(1) + rng.standard_normal(m) * 0.1).astype(np.float32)
    lb = np.full(m, -np.log(m), np.float32)
    got = flashsinkhorn_lse_fused(*dev(x, y, gh, lb), eps, allow_tf32=False).cpu().numpy()
    rows = np.concatenate([rng.choice(n, 96, replace=False), [0, n - 1]])
    want = oracle.lse_shifted_fused(x[rows], y, gh, lb, eps)
    assert np.abs(got[rows] - want).max() <= 3e-6 * np.abs(want).max()


@pytest.mark.parametrize("n,m,d,scale", [(300, 5000, 96, 1.0), (1500, 2100, 128, 1.0),
                                         (260, 1300, 128, 3e3), (260, 1300, 72, 1e-3)])
def test_mat5_wide_rows_on_planes(n, m, d, scale):
    """64 < d <= 128: mat5 runs on fp16 planes with the key operands streamed from LDS step by
    step and both stationary operands in registers (one wavefront per SIMD); several key tiles,
    split keys, and clouds / A in unrelated units."""
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    x, y, a, b, f, g = problem(n, m, d, seed=7)
    x, y = (x * scale).astype(np.float32), (y * scale).astype(np.float32)
    eps = 0.5 * scale * scale
    f = ((f - 2.0) * scale * scale).astype(np.float32)
    g = (g * scale * scale).astype(np.float32)
    A = (np.random.default_rng(8).standard_normal((n, d)) * 50.0 / scale).astype(np.float32)
    want = oracle.mat5(x, y, f, g, A, eps, 0.5)
    got = mat5_sqeuclid(*dev(x, y, f, g, A), eps=eps, cost_scale=0.5)
    assert rel_err(got, want) < RTOL


@pytest.mark.parametrize("scale", [1e-4, 1.0, 3e4])
@pytest.mark.parametrize("d", [64, 200])
def test_symmetric_step_is_scale_robust(scale, d):
    """The default operand mode multiplies fp16 planes of the matrix scaled by a power of two
    taken from its largest magnitude: results must not depend on the units of the clouds, on
    rows far below that maximum, or on a single outlier coordinate far above the rest."""
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    n, m = 300, 257
    x, y, a, b = inputs(101, n, m, d, scale=2.0 / np.sqrt(d))
    x = (x * scale).astype(np.float32)
    y = (y * scale).astype(np.float32)
    x[5] *= 1e-6          # a row 2^-20 below the maximum
    y[7, 3] *= 300.0      # one coordinate far above everything else
    eps = 0.05 * scale * scale
    rng = np.random.default_rng(8)
    fh = (rng.standard_normal(n) * 0.3 * scale * scale).astype(np.float32)
    gh = (rng.standard_normal(m) * 0.3 * scale * scale).astype(np.float32)
    la, lb = np.log(a), np.log(b)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    wf, wg = oracle.symmetric_step(x, y, fh, gh, la, lb, eps, 1.0, 0.5, 1.0, 1.0)
    gf, gg = _symmetric_step_raw(X, Y, F, G, LA, LB, eps, cost_scale=1.0, alpha=0.5,
                                 damping_f=1.0, damping_g=1.0, allow_tf32=False)
    assert rel_err(gf, wf) < RTOL and rel_err(gg, wg) < RTOL


@pytest.mark.parametrize("scale", [1e-4, 1.0, 3e4])
def test_large_d_products_are_scale_robust(scale):
    """The large-d product kernels multiply fp16 planes of x, y, the value matrix and (mat5) A,
    each scaled by a power of two from its largest magnitude, and carry probabilities as fp16
    planes: results must not depend on the units of any of the operands."""
    from flash_sinkhorn_amd.kernels.apply_flash import (
        apply_plan_mat_flashstyle, apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    n, m, d = 150, 700, 200
    x, y, a, b = inputs(103, n, m, d, scale=2.0 / np.sqrt(d))
    x = (x * scale).astype(np.float32)
    y = (y * scale).astype(np.float32)
    y[7, 3] *= 100.0      # one coordinate far above everything else
    eps = 0.3 * scale * scale
    rng = np.random.default_rng(9)
    fh = (rng.standard_normal(n) * 0.3 * scale * scale).astype(np.float32)
    gh = (rng.standard_normal(m) * 0.3 * scale * scale).astype(np.float32)
    la, lb = np.log(a), np.log(b)
    vscale = 1e3 / scale  # values in units unrelated to the clouds
    V = (rng.standard_normal((m, d)) * vscale).astype(np.float32)
    v = (rng.standard_normal(m) * vscale).astype(np.float32)
    z = (rng.random(m) * 1e-3).astype(np.float32)
    X, Y, F, G, LA, LB = dev(x, y, fh, gh, la, lb)
    kw = dict(eps=eps, cost_scale=0.5)
    got = apply_plan_mat_flashstyle(X, Y, F, G, LA, LB, dev(V)[0], axis=1, scale=dev(z)[0], **kw)
    assert rel_err(got, oracle.apply_plan_mat(x, y, fh, gh, la, lb, V, axis=1, scale=z, **kw)) < RTOL
    got = apply_plan_vec_flashstyle(X, Y, F, G, LA, LB, dev(v)[0], axis=1, **kw)
    assert rel_err(got, oracle.apply_plan_vec(x, y, fh, gh, la, lb, v, axis=1, **kw)) < RTOL
    wx, wy = oracle.grad_barycentric(x, y, a, b, fh, gh, eps, cost_scale=0.5)
    gx, gy = grad(X, Y, *dev(a, b), F, G, eps=eps, cost_scale=0.5, allow_tf32=False)
    assert rel_err(gx, wx) < RTOL and rel_err(gy, wy) < RTOL
    A = (rng.standard_normal((n, d)) * vscale).astype(np.float32)
    f5 = fh - 2.0 * scale * scale
    want = oracle.mat5(x, y, f5, gh, A, eps, 0.5)
    got = mat5_sqeuclid(*dev(x, y, f5, gh, A), eps=eps, cost_scale=0.5)
    assert rel_err(got, want) < RTOL


@pytest.mark.parametrize("n,m,d", [(96, 640_000, 64), (8192, 40_000, 160)])
def test_far_tail_of_the_plan_survives_the_fp16_probability_split(n, m, d):
    """One dominant key and a bulk of m - 1 keys at 2^-22 of its weight each (together 0.15 /
    0.01 of the row mass, sitting somewhere else): the products that cut the probabilities into
    fp16 planes (gradient, plan-matrix; d <= 128 and the large-d kernel) must keep that tail.  The
    dominant key comes first, so it is the running maximum of its key chunk from the first tile
    on and the tail sits 22 binades below the largest probability of its row: cut into fp16
    planes as they stand, such probabilities are a few units of the smallest fp16 subnormal and
    all round the same way (1.4 % of the tail, 3e-4 of the answer).  Shapes are chosen so that
    the chunk with the dominant key holds 40,000 keys (16 chunks at d = 64, one at 160).  Not
    tested further down: from 2^-24 on the fp32 accumulator that already holds the dominant
    term rounds the tail's increments (16 keys per MFMA) at its own ulp, in any fp32 scheme."""
    from flash_sinkhorn_amd.kernels.apply_flash import apply_plan_mat_flashstyle
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    rng = np.random.default_rng(11)
    eps, rows = 1.0, slice(0, 64)
    x = (0.01 * rng.standard_normal((n, d))).astype(np.float32)
    y = (0.01 * rng.standard_normal((m, d))).astype(np.float32)
    y[1:] += np.float32(1.0 / np.sqrt(d))
    y[0] -= np.float32(1.0 / np.sqrt(d))
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    g = np.full(m, -22.0 * np.log(2.0) * eps, np.float32)
    g[0] = 0.0
    g += ((y.astype(np.float64) ** 2).sum(1) - (y[0].astype(np.float64) ** 2).sum()).astype(np.float32)
    f = np.zeros(n, np.float32)
    wx, _ = oracle.grad_barycentric(x[rows], y, a[rows], b, f[rows], g, eps)
    # the first 40,000 tail keys carry a visible share of the answer
    w0, _ = oracle.grad_barycentric(x[rows], np.delete(y, np.s_[1:40_000], 0), a[rows],
                                    np.delete(b, np.s_[1:40_000]), f[rows],
                                    np.delete(g, np.s_[1:40_000]), eps)
    assert np.abs(w0 - wx).max() / np.abs(wx).max() > 3e-4
    X, Y, A, B, F, G = dev(x, y, a, b, f, g)
    gx, _ = grad(X, Y, A, B, F, G, eps=eps, allow_tf32=False, compute_grad_y=False)
    assert rel_err(gx[rows], wx) < RTOL
    # plan-matrix product with the same plan: P V, V = key rows
    la, lb = np.log(a), np.log(b)
    f_hat = (f - (x.astype(np.float64) ** 2).sum(1)).astype(np.float32)
    g_hat = (g - (y.astype(np.float64) ** 2).sum(1)).astype(np.float32)
    want = oracle.apply_plan_mat(x[rows], y, f_hat[rows], g_hat, la[rows], lb, y, eps, axis=1)
    got = apply_plan_mat_flashstyle(X, Y, *dev(f_hat, g_hat, la, lb), Y, eps=eps, axis=1)
    assert rel_err(got[rows], want) < RTOL


@pytest.mark.parametrize("mode", ["fp16x2", "fp32_mfma"])
@pytest.mark.parametrize("d", [16, 64, 100, 128, 200])
@pytest.mark.parametrize("lead", [70, 300])
def test_leading_keys_without_weight(monkeypatch, d, lead, mode):
    """The first keys of both clouds carry no weight (log weight -100000, as the reference maps
    them): whole first tiles of every kernel family see logits a hundred thousand base-2 units
    below the rest.  A running maximum subtracted inside the accumulator cost the tiles after
    them their digits (errors of 1e-3); every operation against the fp64 oracle.  Also the two
    ways a key without weight can become a row's starting key: a caller's hint, and the key
    array of prepared planes."""
    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd.kernels._common import log_weights
    from flash_sinkhorn_amd.kernels.apply_flash import (apply_plan_mat_flashstyle,
                                                        apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    monkeypatch.setattr(_lib, "STRICT_OPERANDS", mode)  # the default planes, or fp32 MFMA operands
    rng = np.random.default_rng(7 * d + lead)
    n, m, eps = 1100, 900, 0.05
    x = (rng.standard_normal((n, d)) / np.sqrt(d)).astype(np.float32)
    y = (rng.standard_normal((m, d)) / np.sqrt(d) + 0.1).astype(np.float32)
    a = rng.random(n).astype(np.float32) + 0.5
    b = rng.random(m).astype(np.float32) + 0.5
    a[:lead] = 0
    b[:lead // 2] = 0
    a, b = a / a.sum(), b / b.sum()
    wf, wg = oracle.sinkhorn_symmetric(x, y, a, b, eps=eps, n_iters=6, use_epsilon_scaling=False)[:2]
    X, Y, A, B = dev(x, y, a, b)
    f, g = dev(wf.astype(np.float32), wg.astype(np.float32))
    Fh, Gh = (f - (X * X).sum(1)).contiguous(), (g - (Y * Y).sum(1)).contiguous()
    la, lb = log_weights(A).contiguous(), log_weights(B).contiguous()
    ola, olb = oracle.log_weights(a), oracle.log_weights(b)
    fh, gh = Fh.cpu().numpy(), Gh.cpu().numpy()
    kw = dict(cost_scale=1.0, alpha=1.0, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    want = oracle.symmetric_step(x, y, fh, gh, ola, olb, eps, 1.0, 1.0, 1.0, 1.0)
    tol = 2e-5

    def check(got, exp, what):
        for u, v in zip(got, exp):
            assert rel_err(u, v) < tol, (what, rel_err(u, v))

    check(_symmetric_step_raw(X, Y, Fh, Gh, la, lb, eps, coarse=False, **kw), want, "step")
    planes = mode == "fp16x2"
    if d <= 128 and planes:
        for keys in (None, 0):  # no keys yet; every row's key is key 0, which has no weight
            prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
            if keys is not None:
                prep.best_keys(0).fill_(keys)
                prep.best_keys(1).fill_(keys)
            check(_symmetric_step_raw(X, Y, Fh, Gh, la, lb, eps, coarse=True, prepared=prep, **kw), want,
                  ("coarse step", keys))
    wgrad = oracle.grad_barycentric(x, y, a, b, wf.astype(np.float32), wg.astype(np.float32), eps)[:2]
    check(grad(X, Y, A, B, f, g, eps=eps, allow_tf32=False), wgrad, "gradient")
    if d <= 128 and planes:
        hints = (torch.zeros(n, dtype=torch.int32, device="cuda"), torch.zeros(m, dtype=torch.int32, device="cuda"))
        check(grad(X, Y, A, B, f, g, eps=eps, allow_tf32=False, _seed_keys=hints), wgrad, "hinted gradient")
    V = rng.standard_normal((m, d)).astype(np.float32)
    W = rng.standard_normal((n, d)).astype(np.float32)
    v = rng.standard_normal(m).astype(np.float32)
    check([apply_plan_mat_flashstyle(X, Y, Fh, Gh, la, lb, dev(V)[0], eps=eps, axis=1, allow_tf32=False)],
          [oracle.apply_plan_mat(x, y, fh, gh, ola, olb, V, eps, 1)], "plan.mat")
    check([apply_plan_mat_flashstyle(X, Y, Fh, Gh, la, lb, dev(W)[0], eps=eps, axis=0, allow_tf32=False)],
          [oracle.apply_plan_mat(x, y, fh, gh, ola, olb, W, eps, 0)], "plan^T.mat")
    check([apply_plan_vec_flashstyle(X, Y, Fh, Gh, la, lb, dev(v)[0], eps=eps, axis=1, allow_tf32=False)],
          [oracle.apply_plan_vec(x, y, fh, gh, ola, olb, v, eps, 1)], "plan.vec")
