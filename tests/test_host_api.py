"""Host-side logic and the C-ABI surface; nothing here needs a GPU."""
import ctypes
import os
import re
import warnings

import numpy as np
import pytest
import torch

import oracle
from flash_sinkhorn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "flash_sinkhorn_hip.h")).read()
    declared = set(re.findall(r"\b(fs_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert getattr(handle, name) is not None
    assert _lib.lib().fs_version() >= 1
    assert _lib.lib().fs_error_string(-4) == b"workspace too small"


def test_c_abi_rejects_bad_arguments_before_any_launch():
    L = _lib.lib()
    fake = 0x1000  # never dereferenced: every call below fails validation on the host
    assert L.fs_lse(None, fake, fake, fake, 8, 8, 4, 0.1, 2.0, 1.0, 0, None, 0, None) == -1
    assert L.fs_lse(fake, fake, fake, fake, 0, 8, 4, 0.1, 2.0, 1.0, 0, None, 0, None) == -2
    assert L.fs_lse(fake, fake, fake, fake, 8, 8, 4, 0.0, 2.0, 1.0, 0, None, 0, None) == -3
    assert L.fs_apply_vec(fake, fake, fake, fake, fake, fake, fake, fake, 8, 8, 4, 0.1, 2.0, 2,
                          0, None, 0, None) == -3
    assert L.fs_apply_mat(fake, fake, fake, fake, fake, fake, fake, fake, fake, 8, 8, 4, 4, 0.1,
                          2.0, 0, 0, None, 0, None) == -3  # scale with axis=0
    # sizes whose work-item counts overflow 32-bit launch planning (rows x padded columns / 4)
    assert L.fs_lse(fake, fake, fake, fake, 70_000_000, 8, 128, 0.1, 2.0, 1.0, 0, None, 0, None) == -2
    assert L.fs_lse(fake, fake, fake, fake, 8, 3_000_000, 4096, 0.1, 2.0, 1.0, 0, None, 0, None) == -2
    assert L.fs_workspace_bytes(_lib.OP_LSE, 70_000_000, 8, 128) == 0
    # the entry point with the built-in scratch buffer refuses what does not fit it, on the host
    assert L.fs_workspace_bytes(_lib.OP_SYMMETRIC_STEP, 8192, 8192, 1536) > 48 << 20
    assert L.fs_symmetric_step_noalloc(fake, fake, fake, fake, fake, fake, fake, fake, None, None,
                                       8192, 8192, 1536, 0.1, 0.5, 1.0, 1.0, 2.0, 0, None) == -7
    assert L.fs_error_string(-7) == b"problem too large for the built-in scratch buffer"
    # a split launch without workspace is refused, not launched
    n = m = 50000
    need = L.fs_workspace_bytes(_lib.OP_LSE, n, m, 64)
    assert need > 0
    assert L.fs_lse(fake, fake, fake, fake, n, m, 64, 0.1, 2.0, 1.0, 0, None, 0, None) == -4
    # outputs may not alias inputs in the Jacobi step
    assert L.fs_symmetric_step(fake, fake, fake, fake, fake, fake, fake, fake, None, None, 8, 8,
                               4, 0.1, 0.5, 1.0, 1.0, 2.0, 0, None, 0, None) == -3
    # c-transform: missing output, bad size
    assert L.fs_c_transform(fake, fake, fake, fake, None, 8, 8, 4, 2.0, 0, None, 0, None) == -1
    assert L.fs_c_transform(fake, fake, fake, fake, fake, 8, 0, 4, 2.0, 0, None, 0, None) == -2
    # the multi-step loop: host arrays missing, work vectors aliasing each other, nothing to do
    import ctypes
    one = (ctypes.c_float * 1)(0.1)
    fk = [fake + 0x100 * i for i in range(12)]
    assert L.fs_symmetric_steps(*fk[:10], None, None, 8, 8, 4, None, one, one, one, 1, 2.0, 0,
                                None, 0, None) == -1
    assert L.fs_symmetric_steps(*fk[:6], fk[6], fk[7], fk[6], fk[9], None, None, 8, 8, 4, one, one,
                                one, one, 1, 2.0, 0, None, 0, None) == -3
    assert L.fs_symmetric_steps(*fk[:10], None, None, 8, 8, 4, one, one, one, one, 0, 2.0, 0,
                                None, 0, None) == 0
    # the paired self problems: null schedule, aliased work vectors, bad eps, zero steps
    assert L.fs_self_pair_steps(*fk[:10], None, None, 8, 8, 4, one, None, one, one, one, 1, 2.0, 0,
                                None, 0, None) == -1
    assert L.fs_self_pair_steps(*fk[:6], fk[6], fk[6], fk[8], fk[9], None, None, 8, 8, 4, one, one,
                                one, one, one, 1, 2.0, 0, None, 0, None) == -3
    zero = (ctypes.c_float * 1)(0.0)
    assert L.fs_self_pair_steps(*fk[:10], None, None, 8, 8, 4, one, zero, one, one, one, 1, 2.0, 0,
                                None, 0, None) == -3
    assert L.fs_self_pair_steps(*fk[:10], None, None, 8, 8, 4, one, one, one, one, one, 0, 2.0, 0,
                                None, 0, None) == 0


def test_workspace_is_deterministic_and_zero_for_small_problems():
    L = _lib.lib()
    assert 0 < L.fs_workspace_bytes(_lib.OP_MAT5, 64, 48, 32) < 512 * 1024  # planes (both layouts), no key split
    assert 0 < L.fs_workspace_bytes(_lib.OP_LSE, 64, 48, 32) < 512 * 1024  # 16-bit planes (both layouts) + pad rows
    assert L.fs_workspace_bytes(_lib.OP_GRAD, 64, 48, 20000) == 0          # d beyond the kernels
    a = L.fs_workspace_bytes(_lib.OP_GRAD, 50000, 50000, 64)
    assert a == L.fs_workspace_bytes(_lib.OP_GRAD, 50000, 50000, 64) and a > 0


def test_helpers_match_oracle_closed_forms():
    from flash_sinkhorn_amd.kernels._common import (dampening, epsilon_schedule, log_weights,
                                                     max_diameter)
    assert dampening(0.1, None) == 1.0
    assert dampening(0.1, 1.0) == pytest.approx(1 / 1.1)
    w = torch.tensor([0.5, 0.0, 2.0])
    np.testing.assert_allclose(log_weights(w).numpy(), oracle.log_weights(w.numpy()), rtol=1e-6)
    x = torch.randn(10, 3); y = torch.randn(7, 3) + 1
    assert max_diameter(x, y) == pytest.approx(oracle.max_diameter(x.numpy(), y.numpy()), rel=1e-6)
    assert epsilon_schedule(3.0, 0.1, 0.6) == pytest.approx(oracle.epsilon_schedule(3.0, 0.1, 0.6))
    with pytest.raises(ValueError):
        epsilon_schedule(-1.0, 0.1, 0.5)


def test_shift_helpers():
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        compute_bias_f, compute_bias_g, precompute_flashsinkhorn_inputs,
        shifted_to_standard_potentials, standard_to_shifted_potentials)
    x = torch.randn(6, 4); y = torch.randn(5, 4)
    a = torch.full((6,), 1 / 6); b = torch.full((5,), 1 / 5)
    al, be, ga, de = precompute_flashsinkhorn_inputs(x, y, a, b, 0.2, cost_scale=0.5)
    torch.testing.assert_close(al, 0.5 * (x ** 2).sum(1))
    torch.testing.assert_close(de, 0.2 * b.log())
    g = torch.randn(5); f = torch.randn(6)
    torch.testing.assert_close(compute_bias_f(g, be, de, 0.2), (g - be + de) / 0.2)
    torch.testing.assert_close(compute_bias_g(f, al, ga, 0.2), (f - al + ga) / 0.2)
    fh, gh = standard_to_shifted_potentials(f, g, al, be)
    f2, g2 = shifted_to_standard_potentials(fh, gh, al, be)
    torch.testing.assert_close(f2, f); torch.testing.assert_close(g2, g)


def test_launchers_reject_cpu_tensors_and_bad_shapes():
    from flash_sinkhorn_amd.kernels.apply_flash import (apply_plan_mat_flashstyle,
                                                        apply_plan_vec_flashstyle)
    from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
        flashsinkhorn_lse, flashsinkhorn_lse_fused)
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
        sinkhorn_geomloss_online_grad_sqeuclid as grad)
    x = torch.randn(6, 4); y = torch.randn(5, 4); v = torch.randn(5)
    with pytest.raises(ValueError, match="CUDA"):
        flashsinkhorn_lse(x, y, v, 0.1)
    with pytest.raises(ValueError, match="CUDA"):
        flashsinkhorn_lse_fused(x, y, v, v, 0.1)
    with pytest.raises(ValueError, match="CUDA"):
        grad(x, y, torch.ones(6), torch.ones(5), torch.zeros(6), torch.zeros(5), eps=0.1)
    with pytest.raises(ValueError, match="axis"):
        apply_plan_mat_flashstyle(x, y, torch.zeros(6), v, torch.zeros(6), v, y, eps=0.1, axis=2)
    with pytest.raises(ValueError, match="CUDA"):
        apply_plan_mat_flashstyle(x, y, torch.zeros(6), v, torch.zeros(6), v, y, eps=0.1, axis=1)
    with pytest.raises(AssertionError):
        apply_plan_vec_flashstyle(x, y, torch.zeros(5), v, torch.zeros(6), v, v, eps=0.1, axis=1)
    with pytest.raises(ValueError, match="CUDA"):
        mat5_sqeuclid(x, y, torch.zeros(6), v, x, eps=0.1)


def test_deprecated_names_are_bridged_with_a_warning():
    import flash_sinkhorn_amd.kernels as K
    with warnings.catch_warnings(record=True) as rec:
        warnings.simplefilter("always")
        fn = K.flashsinkhorn_symmetric_step
    assert callable(fn) and any(issubclass(w.category, DeprecationWarning) for w in rec)
    with pytest.raises(AttributeError):
        K.not_a_kernel
    from flash_sinkhorn_amd.kernels.sinkhorn_triton_apply_sqeuclid import mat5_sqeuclid  # noqa


def test_samples_loss_argument_validation():
    from flash_sinkhorn_amd import SamplesLoss
    with pytest.raises(ValueError):
        SamplesLoss("energy")
    with pytest.raises(ValueError):
        SamplesLoss(p=1)
    with pytest.raises(ValueError):
        SamplesLoss(backend="keops")
    with pytest.raises(ValueError):
        SamplesLoss(backend="alternating")  # needs fixed eps
    with pytest.raises(ValueError):
        SamplesLoss(reach=-1.0)
    with pytest.warns(DeprecationWarning):
        assert SamplesLoss(backend="auto").backend == "symmetric"
    L = SamplesLoss(reach=2.0, half_cost=True)
    assert (L.rho_x, L.rho_y, L.rho, L.cost_scale) == (4.0, 4.0, 4.0, 0.5)
    L = SamplesLoss(reach_x=2.0)
    assert (L.rho_x, L.rho_y, L.reach) == (4.0, None, None)
    with pytest.raises(ValueError, match="CUDA"):
        SamplesLoss()(torch.randn(4, 2), torch.randn(3, 2))
    with pytest.raises(TypeError):
        SamplesLoss()(torch.randn(4, 2))
    L = SamplesLoss(use_epsilon_scaling=False, eps=0.1, n_iters=7)
    assert L._eps_list_for_inputs(torch.randn(4, 2), torch.randn(3, 2)) == [0.1] * 7
    L = SamplesLoss(blur=0.1, scaling=0.5, diameter=2.0, n_iters=3)
    assert L._eps_list_for_inputs(None, None) == oracle.epsilon_schedule(2.0, 0.1, 0.5)[:3]


def test_process_args_shapes():
    from flash_sinkhorn_amd.samples_loss import _process_args
    p = _process_args(torch.rand(5, 1), torch.randn(5, 3), torch.rand(4), torch.randn(4, 3),
                      normalize=True)
    assert p.a.shape == (5,) and p.a_view_shape == (5, 1) and p.b_view_shape == (4,)
    assert float(p.a.sum()) == pytest.approx(1.0) and not p.batched
    p = _process_args(torch.randn(2, 5, 3), torch.randn(2, 4, 3), normalize=False)
    assert p.batched and p.a.shape == (2, 5) and float(p.b[0, 0]) == pytest.approx(0.25)
    with pytest.raises(ValueError):
        _process_args(torch.randn(5, 3), torch.randn(4, 2), normalize=True)
    with pytest.raises(ValueError):
        _process_args(torch.rand(6), torch.randn(5, 3), torch.rand(4), torch.randn(4, 3),
                      normalize=True)
    with pytest.raises(ValueError):
        _process_args(torch.randn(2, 5, 3), torch.randn(4, 3), normalize=True)
    with pytest.raises(TypeError):
        _process_args(torch.ones(5, 3, dtype=torch.int32), torch.randn(4, 3), normalize=True)


def test_cg_on_cpu_tensors_matches_oracle_bookkeeping():
    from flash_sinkhorn_amd.cg import conjugate_gradient
    rng = np.random.default_rng(3)
    M = rng.standard_normal((12, 12)); M = M @ M.T + 12 * np.eye(12)
    b = rng.standard_normal(12)
    Mt, bt = torch.from_numpy(M), torch.from_numpy(b)
    x, info = conjugate_gradient(lambda v: Mt @ v, bt, rtol=1e-12, atol=1e-14)
    xo, io = oracle.conjugate_gradient(lambda v: M @ v, b, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(x.numpy(), xo, rtol=1e-9)
    assert (info.cg_converged, info.cg_iters) == (io.cg_converged, io.cg_iters)
    _, info = conjugate_gradient(lambda v: Mt @ v, bt, max_iter=2, rtol=1e-14, atol=0.0)
    assert (not info.cg_converged) and info.cg_iters == 2
    _, info = conjugate_gradient(lambda v: 0 * v, bt)  # zero curvature leaves the loop
    assert not info.cg_converged
    with pytest.raises(ValueError):
        conjugate_gradient(lambda v: v, bt, stabilise_every=-1)
    d = torch.from_numpy(np.diag(M).copy())
    x, _ = conjugate_gradient(lambda v: Mt @ v, bt, preconditioner=lambda r: r / d, x0=bt.clone(),
                              rtol=1e-12, atol=1e-14, stabilise_every=3)
    np.testing.assert_allclose(x.numpy(), xo, rtol=1e-8)


def test_solver_argument_errors():
    from flash_sinkhorn_amd.sinkhorn_solvers import (_resolve_rho, sinkhorn_flashstyle_symmetric)
    assert _resolve_rho(None, 2.0, None, None, None, None) == (4.0, 4.0)
    assert _resolve_rho(1.0, None, None, 5.0, None, None) == (1.0, 5.0)
    with pytest.raises(ValueError):
        _resolve_rho(1.0, 1.0, None, None, None, None)
    with pytest.raises(ValueError):
        _resolve_rho(None, None, 1.0, None, 1.0, None)
    x = torch.randn(4, 2)
    with pytest.raises(ValueError, match="provide eps and n_iters"):
        sinkhorn_flashstyle_symmetric(x, x, torch.ones(4), torch.ones(4),
                                      use_epsilon_scaling=False)
    with pytest.raises(ValueError, match="non-empty"):
        sinkhorn_flashstyle_symmetric(x, x, torch.ones(4), torch.ones(4), eps_list=[])


def test_custom_operators_are_registered_with_shape_inference():
    """torch.ops.flash_sinkhorn_amd.*: every operator exists and its fake implementation gives
    the output shapes and dtypes on meta tensors (no GPU, no library call)."""
    from flash_sinkhorn_amd import torch_ops
    ops = torch.ops.flash_sinkhorn_amd
    for name in torch_ops.OPERATORS:
        assert hasattr(ops, name)
    n, m, d = 7, 5, 3
    mt = lambda *s: torch.empty(*s, device="meta")  # noqa: E731
    x, y = mt(n, d), mt(m, d)
    assert ops.lse(x, y, mt(m), 0.1).shape == (n,)
    assert ops.lse_fused(x, y, mt(m), mt(m), 0.1).shape == (n,)
    f, g = ops.symmetric_step(x, y, mt(n), mt(m), mt(n), mt(m), 0.1)
    assert f.shape == (n,) and g.shape == (m,)
    gx, gy = ops.grad(x, y, mt(n), mt(m), mt(n), mt(m), 0.1)
    assert gx.shape == (n, d) and gy.shape == (m, d)
    assert ops.apply_plan_vec(x, y, mt(n), mt(m), mt(n), mt(m), mt(m), 0.1, 1).shape == (n,)
    assert ops.apply_plan_vec(x, y, mt(n), mt(m), mt(n), mt(m), mt(n), 0.1, 0).shape == (m,)
    assert ops.apply_plan_mat(x, y, mt(n), mt(m), mt(n), mt(m), mt(m, d), 0.1, 1).shape == (n, d)
    assert ops.mat5(x, y, mt(n), mt(m), mt(n, d), 0.1).shape == (n, d)
    c, idx = ops.c_transform(x, y, mt(m))
    assert c.shape == (n,) and idx.dtype == torch.int64 and c.dtype == torch.float32
    out, piz = ops.schur_matvec(x, y, mt(n), mt(m), mt(m), mt(n), mt(m), 0.1)
    assert out.shape == (m,) and piz.shape == (n,)


def test_solvers_refuse_cpu_tensors_before_touching_them():
    import torch
    from flash_sinkhorn_amd.sinkhorn_solvers import (
        sinkhorn_flashstyle_alternating, sinkhorn_flashstyle_symmetric)
    x = torch.randn(10, 3)
    w = torch.full((10,), 0.1)
    with pytest.raises(ValueError, match="CUDA tensors"):
        sinkhorn_flashstyle_symmetric(x, x, w, w, use_epsilon_scaling=False, eps=0.1, n_iters=3)
    with pytest.raises(ValueError, match="CUDA tensors"):
        sinkhorn_flashstyle_alternating(x, x, w, w, eps=0.1, n_iters=3)
