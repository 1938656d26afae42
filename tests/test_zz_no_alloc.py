"""fs_symmetric_step_noalloc (built-in scratch buffer, no workspace argument) through the C ABI
against fs_symmetric_step on a caller-owned workspace: same kernels, same bits.  Two calls in a
row, the second on a smaller problem, so that whatever the first left in the shared buffer is
seen by the second; then the size limit."""
import numpy as np
import pytest
import torch

from tests.golden.recipe import inputs

pytestmark = pytest.mark.gpu


def _both(n, m, d, seed, eps=0.05, alpha=0.5, damp=(1.0, 1.0), shift=False):
    from flash_sinkhorn_amd import _lib
    x, y, a, b = inputs(seed, n, m, d, scale=2.0 / np.sqrt(d))
    rng = np.random.default_rng(seed + 1)
    fh = (-(x * x).sum(1) + 0.1 * rng.standard_normal(n)).astype(np.float32)
    gh = (-(y * y).sum(1) + 0.1 * rng.standard_normal(m)).astype(np.float32)
    X, Y, F, G, LA, LB = [torch.from_numpy(np.ascontiguousarray(t)).cuda()
                          for t in (x, y, fh, gh, np.log(a), np.log(b))]
    SX = (X * X).sum(1).contiguous() if shift else None
    SY = (Y * Y).sum(1).contiguous() if shift else None
    L = _lib.lib()
    st = _lib.stream_of(X)
    fl = _lib.flags(True, False)
    outs = []
    for noalloc in (True, False):
        fo = torch.full((n,), float("nan"), device="cuda")
        go = torch.full((m,), float("nan"), device="cuda")
        head = (X.data_ptr(), Y.data_ptr(), F.data_ptr(), G.data_ptr(), LA.data_ptr(),
                LB.data_ptr(), fo.data_ptr(), go.data_ptr(), _lib.ptr(SX), _lib.ptr(SY), n, m, d,
                eps, alpha, damp[0], damp[1], 2.0, fl)
        if noalloc:
            rc = L.fs_symmetric_step_noalloc(*head, st)
        else:
            ws = _lib.workspace(_lib.OP_SYMMETRIC_STEP, n, m, d, X.device)
            rc = L.fs_symmetric_step(*head, ws.data_ptr(), ws.numel(), st)
        assert rc == 0, L.fs_error_string(rc)
        torch.cuda.synchronize()
        outs.append((fo, go))
    return outs


def test_noalloc_step_equals_workspace_step_twice_in_a_row():
    for n, m, d, seed, kw in [(5000, 4100, 64, 61, {}),
                              (700, 300, 20, 62, dict(damp=(0.8, 0.9), shift=True, alpha=1.0))]:
        (f1, g1), (f0, g0) = _both(n, m, d, seed, **kw)
        assert torch.isfinite(f1).all() and torch.isfinite(g1).all()
        assert torch.equal(f1, f0) and torch.equal(g1, g0)


def test_noalloc_step_rejects_what_does_not_fit():
    from flash_sinkhorn_amd import _lib
    L = _lib.lib()
    n = m = 8192
    d = 1536
    assert L.fs_workspace_bytes(_lib.OP_SYMMETRIC_STEP, n, m, d) > 48 << 20
    t = torch.zeros(8, device="cuda")
    p = t.data_ptr()
    rc = L.fs_symmetric_step_noalloc(p, p, p, p, p, p, p, p, None, None, n, m, d, 0.1, 0.5, 1.0,
                                     1.0, 2.0, 0, _lib.stream_of(t))
    assert rc == -7 and b"scratch" in L.fs_error_string(rc)
