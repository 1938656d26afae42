"""Cache slow fp64 ORACLE results (not reference output) so GPU tests need not recompute them.

``python tests/golden/make_oracle_fixtures.py`` writes ``oracle_config2.npz``: the oracle's
potentials for BASELINE config 2 (n=m=10,000, d=64, eps=0.01, 100 iterations), which takes
minutes of CPU time.  Inputs are regenerated from the seed in the test.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def config2_inputs():
    rng = np.random.default_rng(2)
    n = 10_000
    x = rng.standard_normal((n, 64)).astype(np.float32)
    y = (rng.standard_normal((n, 64)) + 0.5).astype(np.float32)
    a = np.full(n, 1 / n, np.float32)
    return x, y, a


if __name__ == "__main__":
    x, y, a = config2_inputs()
    f, g, fp, gp = oracle.sinkhorn_symmetric(x, y, a, a, use_epsilon_scaling=False, eps=0.01,
                                             n_iters=100, return_prelast=True)
    np.savez_compressed(os.path.join(HERE, "oracle_config2.npz"), f=f, g=g, f_prelast=fp,
                        g_prelast=gp, loss=np.array(oracle.sinkhorn_cost(a, a, f, g, 0.01)))
    print("wrote oracle_config2.npz", float(oracle.sinkhorn_cost(a, a, f, g, 0.01)))
