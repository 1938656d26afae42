"""Hard c-transform (fs_c_transform through the Python mirror) against the fp64 oracle.

Values are held to 1e-5 of the largest magnitude.  Indices must equal the oracle's wherever the
gap between the best and the second-best target exceeds the fp32 rounding of the values, and
must attain the minimum to that rounding everywhere; exact ties resolve to the smaller index.
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

# (n, m, d): d <= 128 runs on fp32 MFMA operands, d > 128 on fp16 planes; split and unsplit keys
SHAPES = [(100, 100, 4), (100, 300, 4), (500, 100, 64), (500, 300, 64), (200, 500, 16),
          (33, 5, 8), (1, 1, 1), (257, 3000, 128), (3000, 2100, 20), (70, 300, 130),
          (100, 1100, 300), (64, 2048, 160), (40, 600, 2048)]


def dev(*arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrs]


def data(n, m, d, seed=0):
    rng = np.random.default_rng(300 + seed)
    return (rng.standard_normal((n, d)).astype(np.float32),
            rng.standard_normal((m, d)).astype(np.float32),
            rng.standard_normal(m).astype(np.float32))


def check_against_oracle(x, y, psi, cs, c, idx):
    want_c, want_idx = oracle.c_transform(x, y, psi, cs)
    c = c.cpu().numpy().astype(np.float64)
    idx = idx.cpu().numpy()
    scale = max(np.abs(want_c).max(), 1.0)
    assert np.abs(c - want_c).max() <= 1e-5 * scale
    assert idx.dtype == np.int64 and idx.min() >= 0 and idx.max() < y.shape[0]
    # the returned target attains the minimum to rounding
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    attained = cs * ((x64 - y64[idx]) ** 2).sum(1) - psi.astype(np.float64)[idx]
    assert np.abs(attained - want_c).max() <= 2e-5 * scale
    # and is the oracle's wherever the runner-up is clearly worse
    C = cs * ((x64[:, None, :] - y64[None, :, :]) ** 2).sum(-1) - psi.astype(np.float64)[None, :]
    if y.shape[0] > 1:
        second = np.partition(C, 1, axis=1)[:, 1]
        clear = (second - want_c) > 1e-4 * scale
        assert np.array_equal(idx[clear], want_idx[clear])
        assert clear.mean() > 0.9


@pytest.mark.parametrize("n,m,d", SHAPES)
@pytest.mark.parametrize("cs", [1.0, 0.5])
def test_values_and_indices(n, m, d, cs):
    from flash_sinkhorn_amd import c_transform_fwd
    x, y, psi = data(n, m, d)
    if d > 128:
        x, y = x / np.sqrt(d / 16), y / np.sqrt(d / 16)  # keep costs O(10) at large d
    c, idx = c_transform_fwd(*dev(x, y, psi), cost_scale=cs, allow_tf32=False)
    check_against_oracle(x, y, psi, cs, c, idx)
    c2, idx2 = c_transform_fwd(*dev(x, y, psi), cost_scale=cs)  # default allow_tf32=True
    check_against_oracle(x, y, psi, cs, c2, idx2)


def test_kernel_entry_returns_inner_minimum():
    from flash_sinkhorn_amd.kernels import c_transform_kernel
    x, y, psi = data(300, 700, 32, seed=1)
    bias = (y * y).sum(1) - psi
    val, idx = c_transform_kernel(*dev(x, y, bias), cost_scale=1.0, allow_tf32=False)
    want_c, want_idx = oracle.c_transform(x, y, psi, 1.0)
    inner = want_c - (x.astype(np.float64) ** 2).sum(1)
    assert np.abs(val.cpu().numpy() - inner).max() <= 1e-5 * np.abs(inner).max()
    assert (idx.cpu().numpy() == want_idx).mean() > 0.99


@pytest.mark.parametrize("m,second", [(96, 64), (5000, 4097), (300, 1)])
def test_ties_resolve_to_the_smaller_index(m, second):
    """Two targets at exactly the same cost, in different lanes, tiles or key splits."""
    from flash_sinkhorn_amd import c_transform_fwd
    y = np.zeros((m, 4), np.float32)
    y[:, 0] = 100.0
    y[0, 0], y[second, 0] = 1.0, -1.0
    x = np.zeros((3, 4), np.float32)
    _, idx = c_transform_fwd(*dev(x, y, np.zeros(m, np.float32)), allow_tf32=False)
    assert idx.tolist() == [0, 0, 0]
    y[0, 0] = 100.0          # now only `second` is near
    _, idx = c_transform_fwd(*dev(x, y, np.zeros(m, np.float32)), allow_tf32=False)
    assert idx.tolist() == [second] * 3


def test_nearest_neighbour_and_cost_scale():
    from flash_sinkhorn_amd import c_transform_fwd
    x, y, _ = data(400, 400, 16, seed=2)
    X, = dev(x)
    c, idx = c_transform_fwd(X, X, torch.zeros(400, device="cuda"), allow_tf32=False)
    assert torch.equal(idx.cpu(), torch.arange(400))
    assert float(c.abs().max()) <= 1e-4
    Y, = dev(y)
    z = torch.zeros(400, device="cuda")
    c1, _ = c_transform_fwd(X, Y, z, cost_scale=1.0)
    ch, _ = c_transform_fwd(X, Y, z, cost_scale=0.5)
    assert float((ch - 0.5 * c1).abs().max()) <= 1e-5 * float(c1.abs().max())


@pytest.mark.parametrize("n,m,d", [(100, 200, 4), (200, 100, 64), (150, 700, 200)])
def test_semi_dual_cost_and_danskin_gradients(n, m, d):
    from flash_sinkhorn_amd import c_transform_cost
    x, y, psi = data(n, m, d, seed=3)
    if d > 128:
        x, y = x / np.sqrt(d / 16), y / np.sqrt(d / 16)
    rng = np.random.default_rng(5)
    a = rng.dirichlet(np.ones(n)).astype(np.float32)
    b = rng.dirichlet(np.ones(m)).astype(np.float32)
    X, Y, P, A, B = dev(x, y, psi, a, b)
    X.requires_grad_(True)
    P.requires_grad_(True)
    loss = c_transform_cost(X, Y, P, cost_scale=0.5, a=A, b=B, allow_tf32=False)
    gx, gp = torch.autograd.grad(3.0 * loss, [X, P])
    L, wx, wp, _ = oracle.c_transform_cost_grads(x, y, psi, a, b, 0.5)
    assert abs(float(loss.detach()) - L) <= 1e-5 * max(abs(L), 1.0)
    # a row whose best two targets are closer than rounding may pick the other one
    row_ok = np.abs(gx.cpu().numpy() / 3.0 - wx).max(1) <= 1e-5 * np.abs(wx).max()
    assert row_ok.mean() > 0.98
    if row_ok.all():
        assert np.abs(gp.cpu().numpy() / 3.0 - wp).max() <= 1e-6
    # uniform default weights
    loss_u = c_transform_cost(X, Y, P, cost_scale=0.5)
    Lu = oracle.c_transform_cost_grads(x, y, psi, np.full(n, 1 / n), np.full(m, 1 / m), 0.5)[0]
    assert abs(float(loss_u.detach()) - Lu) <= 1e-5 * max(abs(Lu), 1.0)


def test_argument_checks():
    from flash_sinkhorn_amd import c_transform_cost, c_transform_fwd
    x, y, psi = (torch.randn(8, 3, device="cuda"), torch.randn(6, 3, device="cuda"),
                 torch.randn(6, device="cuda"))
    with pytest.raises(ValueError):
        c_transform_fwd(x[0], y, psi)
    with pytest.raises(ValueError):
        c_transform_fwd(x, y[:, :2], psi)
    with pytest.raises(ValueError):
        c_transform_fwd(x, y, psi[:5])
    with pytest.raises(ValueError):
        c_transform_fwd(x.cpu(), y, psi)
    with pytest.raises(ValueError):
        c_transform_fwd(x, y[:0], psi[:0])
    with pytest.raises(NotImplementedError):
        c_transform_fwd(x, y.clone().requires_grad_(True), psi)
    yg = y.clone().requires_grad_(True)
    with pytest.raises(NotImplementedError):
        c_transform_cost(x.clone().requires_grad_(True), yg, psi)
    with pytest.raises(ValueError):
        c_transform_cost(x, y, psi, a=torch.full((8,), 0.125, device="cuda", requires_grad=True))
    with pytest.raises(ValueError):
        c_transform_cost(x, y, psi, b=torch.ones(5, device="cuda"))
