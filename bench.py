"""Headline benchmark: ms per 100 symmetric Sinkhorn iterations, n=m=50,000, d=64, fp32.

One "step" is one full solve, ``sinkhorn_flashstyle_symmetric(use_epsilon_scaling=False,
eps=0.01, n_iters=100, last_extrapolation=True, allow_tf32=False)`` = 102 double
log-sum-exp launches, on a seeded 8-component Gaussian mixture per cloud with
uniform weights, inputs already resident in HBM.  Prints ONE JSON line.

Operand modes of the log-sum-exp kernel (results are fp32 in all of them):
  strict (default, allow_tf32=False)  two fp16 planes per operand (22 significand bits) of the
                                      power-of-two scaled matrix, three MFMA products, fp32
                                      accumulate: error <= that of fp32 MFMA operands
  bf16x3 (--mode bf16x3)              three bf16 planes, six products: same accuracy class
  fp32_mfma (--mode fp32_mfma)        fp32 operands on v_mfma_f32_32x32x2_f32
  reduced (--mode reduced)            two bf16 planes, three products (allow_tf32=True)

roofline: one symmetric-step launch does 4*n*m*d algorithmic matrix flop (both
half-updates) plus 2*n*m exp2; its duration is measured here with HIP events on the
launch stream.  The split modes execute 3 (fp16x2, reduced) or 6 (bf16x3) 16-bit MFMA
products per algorithmic product, so the algorithmic rate is priced against the published
2516.6 TFLOP/s fp16/bf16 peak divided by that factor (838.9 or 419.4 TFLOP/s; 157.3 for fp32
MFMA operands); the ratio to the fp32 MFMA peak and the serial / overlapped MFMA+exp roofline
times of the whole 102-step solve are reported next to it.
The solver groups rows by k-means cluster and picks, by timing a few steps, between the plain
kernel and the one that tests a tile after its hi*hi plane product; the roofline launch is
timed on the same row order and variant (reported under roofline.tile_skip).
cpu_baseline: the numpy oracle's symmetric step (fp32) timed on the host cores on a
bounded sample and scaled to the metric's unit.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

N, M, D = 50_000, 50_000, 64
EPS = 0.01
ITERS = 100
MODES = ["strict", "bf16x3", "fp32_mfma", "reduced"]
FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2516.6
EXP2_PER_S = 18.6e12  # v_exp_f32 lanes per second measured on the box (half rate)
# Memory-side bytes per lse2_kernel launch of the default workload, per operand mode, from two
# rocprofv3 --pmc runs (FETCH_SIZE 113,782 KiB x 2.0, WRITE_SIZE 12,510 KiB x 1.0 for the kernel
# variant with the coarse tile test, 112,309 / 12,509 for the plain one; the factors
# are what the same counters read for the 256 MiB copy of --copy-calibration: half the bytes
# copied and all of them).  Not measured for the other modes.
MEASURED_TRAFFIC_BYTES = {"strict": int((113782 * 2.0 + 12510) * 1024)}


def gmm_cloud(rng, n, d, k=8):
    import numpy as np

    means = rng.standard_normal((k, d)) * 2.0
    comp = rng.integers(0, k, size=n)
    return (means[comp] + rng.standard_normal((n, d))).astype(np.float32)


def make_inputs(n, m, d, seed=3):
    import numpy as np

    rng = np.random.default_rng(seed)
    x = gmm_cloud(rng, n, d)
    y = gmm_cloud(rng, m, d)
    a = np.full(n, 1.0 / n, np.float32)
    b = np.full(m, 1.0 / m, np.float32)
    return x, y, a, b


def cpu_baseline(x, y, a, b, budget_s=20.0):
    """Oracle symmetric steps (fp32 numpy) on a row sample, scaled to ms/100 iterations."""
    import numpy as np

    import oracle

    n, m = x.shape[0], y.shape[0]
    rows = min(n, 4096)
    la, lb = np.log(a), np.log(b)
    fh = -(x.astype(np.float32) ** 2).sum(1)
    gh = -(y.astype(np.float32) ** 2).sum(1)
    done, t0 = 0, time.perf_counter()
    for i0 in range(0, n, rows):
        i1 = min(n, i0 + rows)
        # one half-update for these query rows against all m keys, and the mirrored one
        oracle.lse_shifted_fused(x[i0:i1], y, gh, lb, EPS, dtype=np.float32)
        oracle.lse_shifted_fused(y[i0:i1], x, fh, la, EPS, dtype=np.float32)
        done += i1 - i0
        el = time.perf_counter() - t0
        if el > budget_s:
            break
    frac = done / n  # fraction of one full symmetric iteration that was timed
    ms_per_100 = el / frac * (ITERS + 2) * 1e3
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    return {
        "value": ms_per_100, "unit": "ms per 100 symmetric iterations", "cores": cores,
        "kind": "port",
        "sample": f"{done} of {n} query rows of each half-update against all {m} keys "
                  f"({el:.1f} s of the numpy fp32 oracle, BLAS threads = host default), scaled "
                  "to 102 steps",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n", type=int, default=N)
    ap.add_argument("--m", type=int, default=M)
    ap.add_argument("--d", type=int, default=D)
    ap.add_argument("--mode", choices=MODES, default="strict")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-modes", action="store_true",
                    help="skip the one-launch timings of the other operand modes")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device copy: under rocprofv3 --pmc its "
                         "FETCH_SIZE / WRITE_SIZE give the counters' scale factors")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from flash_sinkhorn_amd import _lib
    from flash_sinkhorn_amd import sinkhorn_solvers as solvers
    from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_symmetric
    from flash_sinkhorn_amd.kernels._common import log_weights
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_step_raw

    n, m, d = args.n, args.m, args.d
    x, y, a, b = make_inputs(n, m, d)
    dev = torch.device("cuda:0")
    X, Y, A, B = (torch.from_numpy(t).to(dev) for t in (x, y, a, b))

    def set_mode(mode):
        _lib.STRICT_OPERANDS = {"fp32_mfma": "fp32_mfma", "bf16x3": "bf16x3"}.get(mode, "fp16x2")
        return mode == "reduced"  # allow_tf32

    def solve(mode):
        tf32 = set_mode(mode)
        return sinkhorn_flashstyle_symmetric(
            X, Y, A, B, use_epsilon_scaling=False, eps=EPS, n_iters=ITERS,
            last_extrapolation=True, allow_tf32=tf32)

    for _ in range(args.warmup):
        solve(args.mode)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        f, g = solve(args.mode)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # dominant kernel: one symmetric-step launch, timed with events on the launch stream
    alpha = (X * X).sum(1).contiguous()
    beta = (Y * Y).sum(1).contiguous()
    la, lb = log_weights(A).contiguous(), log_weights(B).contiguous()
    fh, gh = (f - alpha).contiguous(), (g - beta).contiguous()

    # the launch as the solve runs it: rows in the solver's cluster order and the kernel variant
    # it chose (main mode only; the other modes have neither)
    solve_info = dict(solvers.LAST_SOLVE)
    ordered = None
    if solve_info["cluster_order"]:
        px, py = solvers._cluster_order(X), solvers._cluster_order(Y)
        ordered = (X[px].contiguous(), Y[py].contiguous(), fh[px].contiguous(),
                   gh[py].contiguous(), la[px].contiguous(), lb[py].contiguous())

    def launch_ms(mode, reps=20, as_solved=False, coarse=False):
        tf32 = set_mode(mode)
        kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=tf32)
        ops = (X, Y, fh, gh, la, lb)
        if as_solved and ordered is not None:
            ops = ordered
            kw["coarse"] = coarse
        _symmetric_step_raw(*ops, EPS, **kw)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            _symmetric_step_raw(*ops, EPS, **kw)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    flop = 4.0 * n * m * d
    products = {"strict": 3, "bf16x3": 6, "reduced": 3, "fp32_mfma": 0}
    dtypes = {"strict": "fp16x2-planes/fp32-accumulate (fp32-grade)",
              "bf16x3": "bf16x3-planes/fp32-accumulate (fp32-grade)", "fp32_mfma": "f32",
              "reduced": "bf16x2-planes/fp32-accumulate"}

    def roofline_for(mode, ms):
        achieved = flop / (ms * 1e-3) / 1e12
        peak = BF16_MFMA_PEAK_TFLOPS / products[mode] if products[mode] else FP32_MFMA_PEAK_TFLOPS
        r = {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
             "frac": achieved / peak,
             "traffic": MEASURED_TRAFFIC_BYTES.get(mode) if (n, m, d) == (N, M, D) else None,
             "kernel": "one symmetric step (both half-updates) = absmax + split_planes + "
                       "lse2_kernel + finish_kernel; 4*n*m*d algorithmic flop",
             "launch_ms": ms, "exp_per_s": 2.0 * n * m / (ms * 1e-3),
             "frac_of_fp32_mfma_peak": achieved / FP32_MFMA_PEAK_TFLOPS}
        if products[mode]:
            r["peak_note"] = (f"published 16-bit MFMA peak {BF16_MFMA_PEAK_TFLOPS} TFLOP/s / "
                              f"{products[mode]} products per fp32-grade product")
        # MFMA + exp roofline of the whole solve (102 steps), exp2 at the measured 18.6e12 /s
        t_mfma = (ITERS + 2) * flop / (peak * 1e12) * 1e3
        t_exp = (ITERS + 2) * 2.0 * n * m / EXP2_PER_S * 1e3
        r["mfma_exp_roofline_ms"] = {"mfma": t_mfma, "exp": t_exp, "serial": t_mfma + t_exp,
                                     "overlapped": max(t_mfma, t_exp)}
        return r

    main_ms = launch_ms(args.mode, as_solved=True, coarse=solve_info["coarse_test"])
    line = {
        "metric": "ms per 100 symmetric Sinkhorn iterations (n=m=50k, d=64, fp32)",
        "value": ms_per_step, "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": dtypes[args.mode],
        "data": "synthetic",
        "config": {"workload": f"balanced symmetric FlashSinkhorn, n={n}, m={m}, d={d}, seeded "
                               "8-component Gaussian mixtures, uniform weights, eps=0.01, "
                               "100 iterations + init + extrapolation = 102 steps",
                   "operand_mode": args.mode,
                   "loss": float((A * f).sum() + (B * g).sum())},
        "roofline": roofline_for(args.mode, main_ms),
    }
    line["roofline"]["frac_of_serial_mfma_exp_roofline"] = (
        line["roofline"]["mfma_exp_roofline_ms"]["serial"] / ms_per_step)
    # The kernel leaves out the exponentials of 32x32 logits tiles that lie 2^40 below their
    # rows' running maxima (exact in fp32; how many there are depends on the data: about 60 %
    # on this workload).  The same launch with every exponential computed, for comparison:
    _lib.TILE_SKIP = False
    ms_noskip = launch_ms(args.mode, reps=10)
    _lib.TILE_SKIP = True
    line["roofline"]["tile_skip"] = {
        "enabled": True, "launch_ms_with_every_exp": ms_noskip,
        "rows_in_cluster_order": solve_info["cluster_order"],
        "coarse_test": solve_info["coarse_test"],
        "launch_ms_caller_order_no_coarse_test": launch_ms(args.mode, reps=10),
        "note": "tiles whose logits all lie more than 2^40 below the running row maxima skip "
                "their exp2 (no change to fp32 sums); with coarse_test such a tile is recognised "
                "after its hi*hi plane product (bound on the cross products) and skips the other "
                "8 of its 12 MFMAs too, so the executed MFMA flop are fewer than the algorithmic "
                "flop `achieved` counts; launch_ms_with_every_exp computes everything"}
    if not args.no_other_modes:
        others = {}
        for mode in MODES:
            if mode != args.mode:
                ms = launch_ms(mode, reps=10)
                rf = roofline_for(mode, ms)
                others[mode] = {"launch_ms": ms, "ms_per_100_iters_est": ms * (ITERS + 2),
                                "achieved": rf["achieved"], "peak": rf["peak"], "frac": rf["frac"]}
        line["other_operand_modes"] = others
        set_mode(args.mode)
    if args.copy_calibration:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(x, y, a, b)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
