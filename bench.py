"""Headline benchmark: ms per 100 symmetric Sinkhorn iterations, n=m=50,000, d=64, fp32.

One "step" is one full solve, ``sinkhorn_flashstyle_symmetric(use_epsilon_scaling=False,
eps=0.01, n_iters=100, last_extrapolation=True, allow_tf32=False)`` = 102 double
log-sum-exp launches, on a seeded 8-component Gaussian mixture per cloud with
uniform weights, inputs already resident in HBM.  Prints ONE JSON line.

Operand modes (results are fp32 in both):
  strict (default)          two fp16 planes per operand (22 significand bits) of the power-of-two
                            scaled matrix, three MFMA products, fp32 accumulate: error <= that
                            of fp32 MFMA operands; allow_tf32=True runs the same kernels
  fp32_mfma (--mode ...)    fp32 operands on v_mfma_f32_32x32x2_f32

roofline (dominant kernel: lse_coarse_kernel, or lse2_kernel when the plain variant runs; one
launch = both half-updates of a symmetric step, with its small merge kernel): the launch is timed
with HIP events on the launch stream, on prepared operand planes and with the kernel variant
the solve used, after the eight launches in which the rows' starting keys settle.
  algorithmic work of a launch   4*n*m*d matrix flop (2*n*m*d per half-update) + 2*n*m exp2
  executed work                  the fp16 two-plane mode runs three 16-bit MFMA products per
                                 algorithmic product; the variant with the coarse tile test ends
                                 a 32x32 tile after its hi*hi product (1 of 3, plus one MFMA for
                                 the bias bound) when no logit of it can matter, and counts such
                                 tiles on the device
  roofline.achieved              EXECUTED 16-bit MFMA flop / launch time, against the published
                                 dense fp16 peak (2516.6 TFLOP/s); roofline.frac = their ratio.
                                 roofline.algorithmic_tflops = 4*n*m*d / launch time is what a
                                 user gets (it counts flop the coarse test never ran).
The solver lets the device decide, from the share of tiles that end at the coarse test, which
kernel variant runs; value_plain_kernel_ms is the same solve with the plain variant on every
tile, which is what a plan too flat for the test to end anything costs.  Once its potentials
have settled the plain variant takes both sides' sums of a step from one sweep over the logits
(lse_sweep_kernel, half the MFMA and exp2 work; roofline.other_launches.one_sweep_kernel);
value_two_sided_kernel_ms is the same solve with that form switched off (lse2_kernel twice over
the logits in every step).
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
MODES = ["strict", "fp32_mfma"]
FP32_MFMA_PEAK_TFLOPS = 157.3
F16_MFMA_PEAK_TFLOPS = 2516.6
EXP2_PER_S = 18.6e12  # v_exp_f32 lanes per second measured on the box (half rate)
# Memory-side bytes per lse_sparse_kernel launch of the default workload, from two rocprofv3 --pmc
# runs (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch, each times the factor that the same
# counter shows for the 256 MiB device copy of --copy-calibration); see profiles/.
MEASURED_TRAFFIC_BYTES = {"strict": int((134600 * 2.0 + 15550) * 1024)}


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


def cpu_model():
    """Model name plus the family / model / stepping numbers of /proc/cpuinfo (virtual machines
    often shorten the name to the vendor's series)."""
    want = ("model name", "cpu family", "model", "stepping")
    got = {}
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                key, _, val = line.partition(":")
                key = key.strip().lower()
                if key in want and key not in got:
                    got[key] = val.strip()
                if len(got) == len(want):
                    break
    except OSError:
        pass
    if not got:
        return "unknown"
    return (f"{got.get('model name', 'unknown')} (family {got.get('cpu family', '?')}, model "
            f"{got.get('model', '?')}, stepping {got.get('stepping', '?')})")


def blas_threads(cores):
    """Pin the BLAS / OpenMP pools numpy uses to the host cores this process may run on, and
    say how many threads they then have."""
    try:
        from threadpoolctl import threadpool_info, threadpool_limits
        threadpool_limits(limits=cores)
        return max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:  # noqa: BLE001 - a reported figure only
        return None


def cpu_baseline(x, y, a, b, budget_s=20.0):
    """Oracle symmetric steps (fp32 numpy) on a row sample, scaled to ms/100 iterations."""
    import numpy as np

    import oracle

    n, m = x.shape[0], y.shape[0]
    rows = min(n, 4096)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    threads = blas_threads(cores)
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
    return {
        "value": ms_per_100, "unit": "ms per 100 symmetric iterations", "cores": cores,
        "blas_threads": threads, "cpu_model": cpu_model(), "kind": "port",
        "sample": f"{done} of {n} query rows of each half-update against all {m} keys "
                  f"({el:.1f} s of the numpy fp32 oracle, BLAS pool limited to {cores} threads), "
                  "scaled to 102 steps",
    }


def cpu_baseline_other_configs():
    """The numpy fp32 oracle on the host cores at the other four benchmark configurations, per
    unit of work (--cpu-configs; about three minutes).  Seeds and shapes as in BASELINE's
    configurations; every figure is wall time of the dense / row-chunked oracle."""
    import numpy as np

    import oracle

    def timed(fn, reps=1):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2] * 1e3

    out = {}
    f32 = np.float32
    # configuration 1: n = m = 2000, d = 3, eps = 0.01, half cost, 100 iterations, the three
    # solves of a debiased loss, median of 3
    rng = np.random.default_rng(1)
    x, y = rng.standard_normal((2000, 3)).astype(f32), rng.standard_normal((2000, 3)).astype(f32)
    a = np.full(2000, 1 / 2000, f32)
    kw = dict(use_epsilon_scaling=False, eps=0.01, n_iters=100, cost_scale=0.5, dtype=f32)

    def c1():
        for p, q in ((x, y), (x, x), (y, y)):
            oracle.sinkhorn_symmetric(p, q, a, a, **kw)
    out["c1_debiased_solves_100_iters_ms"] = timed(c1, 3)
    # configuration 2: n = m = 10,000, d = 64: 5 symmetric iterations timed, scaled to 100 + 2
    rng = np.random.default_rng(2)
    x = rng.standard_normal((10000, 64)).astype(f32)
    y = (rng.standard_normal((10000, 64)) + 0.5).astype(f32)
    a = np.full(10000, 1e-4, f32)
    la = np.log(a)
    fh, gh = -(x * x).sum(1), -(y * y).sum(1)

    def c2():
        for _ in range(5):
            oracle.symmetric_step(x, y, fh, gh, la, la, 0.01, 1.0, 0.5, 1.0, 1.0, dtype=f32)
    out["c2_xy_solve_100_iters_ms_from_5_steps"] = timed(c2) / 5 * 102
    # configuration 4: n = 20,000, m = 30,000, d = 128: one alternating iteration (two half-updates)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((20000, 128)).astype(f32)
    y = (1.5 * rng.standard_normal((30000, 128))).astype(f32)
    a = rng.dirichlet(np.ones(20000)).astype(f32)
    b = (1.3 * rng.dirichlet(np.ones(30000))).astype(f32)
    out["c4_one_alternating_iteration_ms"] = timed(lambda: oracle.sinkhorn_alternating(
        x, y, a, b, eps=0.0025, n_iters=1, reach=1.0, dtype=f32))
    # configuration 5: n = m = 8192, d = 1536: one gradient (both sides), one plan-vector product
    # pair (the matrix-vector work of one CG iteration)
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((8192, 1536)) / np.sqrt(1536)).astype(f32)
    y = (rng.standard_normal((8192, 1536)) / np.sqrt(1536)).astype(f32)
    a = np.full(8192, 1 / 8192, f32)
    la = np.log(a)
    fz = np.zeros(8192, f32)
    out["c5_one_gradient_ms"] = timed(lambda: oracle.grad_barycentric(x, y, a, a, fz, fz, 0.25,
                                                                      dtype=f32))
    fh, gh = -(x * x).sum(1), -(y * y).sum(1)
    v = rng.standard_normal(8192).astype(f32)

    def c5_cg():
        w = oracle.apply_plan_vec(x, y, fh, gh, la, la, v, 0.25, 1, dtype=f32)
        oracle.apply_plan_vec(x, y, fh, gh, la, la, w, 0.25, 0, dtype=f32)
    out["c5_one_cg_iteration_matvecs_ms"] = timed(c5_cg)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    out.update(cores=cores, blas_threads=blas_threads(cores), cpu_model=cpu_model(), kind="port",
               note="numpy fp32 oracle, BLAS pool limited to the core count")
    return out


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
    ap.add_argument("--cpu-configs", action="store_true",
                    help="also time the CPU oracle at the other four benchmark configurations "
                         "(per unit of work; about three minutes)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the comparison timings (other operand mode, data-independent "
                         "solve, every-exponential launch, 101-step solve)")
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
    from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import _symmetric_steps_raw

    n, m, d = args.n, args.m, args.d
    x, y, a, b = make_inputs(n, m, d)
    dev = torch.device("cuda:0")
    X, Y, A, B = (torch.from_numpy(t).to(dev) for t in (x, y, a, b))

    def set_mode(mode):
        _lib.STRICT_OPERANDS = "fp32_mfma" if mode == "fp32_mfma" else "fp16x2"

    def solve(mode, info=None, **kw):
        set_mode(mode)
        opts = dict(use_epsilon_scaling=False, eps=EPS, n_iters=ITERS, last_extrapolation=True,
                    allow_tf32=False, solve_info=info)
        opts.update(kw)
        return sinkhorn_flashstyle_symmetric(X, Y, A, B, **opts)

    def timed_solves(reps, warm, **kw):
        for _ in range(warm):
            solve(args.mode, **kw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            out = solve(args.mode, **kw)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps, out

    solve_info = {}
    for _ in range(args.warmup):
        solve(args.mode)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        f, g = solve(args.mode, solve_info)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    chosen = solve_info["prepared"].variant_state() if solve_info["coarse"] == "auto" else None
    coarse_ran = (solve_info["coarse"] is True
                  or (chosen is not None and not chosen["plain_selected"]))

    # dominant kernel: symmetric-step launches on prepared operand planes with the kernel variant
    # of the solve, timed with events on the launch stream
    alpha = (X * X).sum(1).contiguous()
    beta = (Y * Y).sum(1).contiguous()
    la, lb = log_weights(A).contiguous(), log_weights(B).contiguous()
    fh, gh = (f - alpha).contiguous(), (g - beta).contiguous()
    ops = (X, Y, fh, gh, la, lb)

    def launch_ms(mode, coarse=False, reps=20, sweep=True):
        """(ms per launch, device counters of the coarse variant over the timed launches);
        sweep=False: steps of the plain variant stay on the two-sided kernel"""
        set_mode(mode)
        _lib.SWEEP = sweep
        prep = _lib.PreparedOperands(ops[0], ops[1], _lib.flags(True, False))
        kw = dict(cost_scale=1.0, allow_tf32=False, prepared=prep, coarse=coarse)
        steps = [(EPS, 0.5, 1.0, 1.0)] * reps
        # the launches that take the decision, in which the rows' starting keys settle and after
        # which the kernel with the coarse tile test runs in its sparse form
        _symmetric_steps_raw(*ops, steps[:16], **kw)
        torch.cuda.synchronize()
        before = prep.variant_state()
        stream = torch.cuda.current_stream(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        _symmetric_steps_raw(*ops, steps, **kw)
        e1.record(stream)
        torch.cuda.synchronize()
        after = prep.variant_state()
        counts = {k: (after[k] - before[k]) / reps
                  for k in ("tiles_ended", "tiles_tested", "tiles_skipped")}
        counts["plain_selected"] = after["plain_selected"]
        counts["one_sweep"] = bool(after["sweep_next"]) and (coarse is False or after["plain_selected"])
        _lib.SWEEP = True
        return e0.elapsed_time(e1) / reps, counts

    flop = 4.0 * n * m * d
    dp = 16 if d <= 16 else (32 if d <= 32 else (64 if d <= 64 else 128))
    tiles_all = 2.0 * -(-n // 32) * -(-m // 32)  # 32 x 32 logits tiles of a launch, both sides
    flop_per_tile_product = 2.0 * 32 * 32 * dp   # one plane product of one tile

    def roofline_for(mode, ms, counts):
        r = {"bound": "mfma", "unit": "TFLOP/s",
             "kernel": ("lse_coarse_kernel" if counts is not None and counts["tiles_tested"] > 0
                        and not counts["plain_selected"] else "lse2_kernel")
                       + " (+ its merge kernel): one launch = both half-updates of a symmetric "
                         "step on prepared operand planes; algorithmic work 4*n*m*d flop + 2*n*m "
                         "exp2",
             "launch_ms": ms, "algorithmic_tflops": flop / (ms * 1e-3) / 1e12,
             "exp_per_s": 2.0 * n * m / (ms * 1e-3)}
        if mode == "fp32_mfma":
            r.update(achieved=r["algorithmic_tflops"], peak=FP32_MFMA_PEAK_TFLOPS,
                     peak_note="published dense fp32 MFMA peak; executed = algorithmic flop")
        else:
            # three plane products per tile in the plain kernel.  The variant with the coarse tile
            # test runs, for every tile it visits, the hi*hi product plus one more 16-column MFMA
            # step that carries the bias bound, and the two cross products only for tiles that go
            # on; its sparse form does not visit tiles whose carried margin still holds.
            products = 3.0 * tiles_all
            exps = 2.0 * n * m
            if counts is not None and counts.get("one_sweep"):
                # both sides from one sweep over the logits: half the tiles, half the exponentials
                products, exps = products / 2, exps / 2
                r["kernel"] = r["kernel"].replace("lse2_kernel", "lse_sweep_kernel")
            if counts is not None and counts["tiles_tested"] > 0 and not counts["plain_selected"]:
                went_on = 1.0 - counts["tiles_ended"] / counts["tiles_tested"]
                visited = 1.0 - counts["tiles_skipped"] / counts["tiles_tested"]
                products = tiles_all * (visited * (1.0 + 16.0 / dp) + 2.0 * went_on)
                r["coarse_test"] = {
                    "share_of_tiles_not_visited": 1.0 - visited,
                    "share_of_tiles_visited_only_to_end_again": visited - went_on,
                    "share_of_tiles_in_full": went_on,
                    "mfma_products_per_tile": products / tiles_all}
                exps = tiles_all * went_on * 1024.0  # only tiles in full run their exponentials
                if visited < 0.5:
                    r["kernel"] = r["kernel"].replace("lse_coarse_kernel", "lse_coarse_kernel, sparse form")
            executed = products * flop_per_tile_product
            r.update(achieved=executed / (ms * 1e-3) / 1e12, peak=F16_MFMA_PEAK_TFLOPS,
                     executed_flop_per_launch=executed, executed_exp2_per_launch=exps,
                     peak_note="published dense fp16 MFMA peak; achieved counts the 16-bit MFMA "
                               "flop the launch executed (three plane products per algorithmic "
                               "product, one for tiles that end at the coarse test, none for "
                               "tiles not visited, padding of d to the MFMA width included)")
        r["frac"] = r["achieved"] / r["peak"]
        r["frac_algorithmic"] = r["algorithmic_tflops"] / r["peak"]  # counts work the launch did not have to do
        r["traffic"] = MEASURED_TRAFFIC_BYTES.get(mode) if (n, m, d) == (N, M, D) else None
        return r

    as_solved = "auto" if solve_info["coarse"] == "auto" else bool(solve_info["coarse"])
    main_ms, main_counts = launch_ms(args.mode, coarse=as_solved)
    line = {
        "metric": "ms per 100 symmetric Sinkhorn iterations (n=m=50k, d=64, fp32)",
        "value": ms_per_step, "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if args.mode == "fp32_mfma" else
                 "fp16x2-planes/fp32-accumulate (fp32-grade)",
        "data": "synthetic",
        "config": {"workload": f"balanced symmetric FlashSinkhorn, n={n}, m={m}, d={d}, seeded "
                               "8-component Gaussian mixtures, uniform weights, eps=0.01, "
                               "100 iterations + init + extrapolation = 102 steps",
                   "operand_mode": args.mode,
                   "kernel_variant": "coarse tile test" if coarse_ran else "plain",
                   "variant_chosen_by": ("device counters" if solve_info["coarse"] == "auto"
                                         else "caller"),
                   "loss": float((A * f).sum() + (B * g).sum())},
        "roofline": roofline_for(args.mode, main_ms, main_counts),
    }
    rf = line["roofline"]
    # MFMA + exp2 roofline of the timed launch for the work it EXECUTED (16-bit MFMA flop at the
    # published peak, exponentials at the measured v_exp_f32 rate): what the matrix and the
    # transcendental pipe would need for that work one after the other, against the launch time
    t_mfma = rf["achieved"] * main_ms / rf["peak"]
    t_exp = rf.get("executed_exp2_per_launch", 2.0 * n * m) / EXP2_PER_S * 1e3
    rf["mfma_exp_roofline_of_executed_work_ms"] = {
        "mfma": t_mfma, "exp2": t_exp, "serial": t_mfma + t_exp, "overlapped": max(t_mfma, t_exp)}
    rf["frac_of_serial_mfma_exp_roofline"] = (t_mfma + t_exp) / main_ms

    if not args.no_extras:
        # the plan-independent figure: the plain kernel on every tile
        forced = solvers.COARSE_TEST
        solvers.COARSE_TEST = False
        line["value_plain_kernel_ms"], _ = timed_solves(max(2, args.steps // 2), 1)
        # (value_two_sided_kernel_ms, below: the same without the one-sweep form)
        solvers.COARSE_TEST = forced
        # the 101-step variant (no extrapolation step) that the reference's README times
        line["value_without_last_extrapolation_ms"], _ = timed_solves(
            max(2, args.steps // 2), 1, last_extrapolation=False)
        solvers.COARSE_TEST = False
        _lib.SWEEP = False
        line["value_two_sided_kernel_ms"], _ = timed_solves(max(2, args.steps // 2), 1)
        _lib.SWEEP = True
        solvers.COARSE_TEST = forced
        sweep_ms, sweep_counts = launch_ms(args.mode)
        plain_ms, _ = launch_ms(args.mode, sweep=False)
        _lib.TILE_SKIP = False
        every_exp_ms, _ = launch_ms(args.mode, reps=10, sweep=False)
        _lib.TILE_SKIP = True
        rf["other_launches"] = {
            "one_sweep_kernel": {
                "launch_ms": sweep_ms, "ran": sweep_counts["one_sweep"],
                **{k: v for k, v in roofline_for(args.mode, sweep_ms, sweep_counts).items()
                   if k in ("achieved", "frac", "algorithmic_tflops")},
                "note": "plain variant on settled potentials: lse_sweep_kernel takes both sides' "
                        "sums from one sweep over the logits (half the MFMA and exp2 work of the "
                        "two-sided launch; achieved counts the executed half)"},
            "plain_kernel": {
                "launch_ms": plain_ms, **{k: v for k, v in roofline_for(
                    args.mode, plain_ms, None).items() if k in ("achieved", "frac",
                                                                "algorithmic_tflops")}},
            "plain_kernel_every_exp": {
                "launch_ms": every_exp_ms, **{k: v for k, v in roofline_for(
                    args.mode, every_exp_ms, None).items() if k in ("achieved", "frac",
                                                                    "algorithmic_tflops")}},
            "note": "the plain kernel runs every MFMA and leaves out only the exp2 of tiles "
                    "whose logits all lie 2^40 below their rows' running maxima (exact in "
                    "fp32); every_exp computes those too"}
        other = "fp32_mfma" if args.mode == "strict" else "strict"
        o_ms, _ = launch_ms(other, reps=5)
        orf = roofline_for(other, o_ms, None)
        set_mode(other)
        forced = solvers.COARSE_TEST
        solvers.COARSE_TEST = False if other == "fp32_mfma" else forced
        saved_mode, args.mode = args.mode, other
        o_solve_ms, _ = timed_solves(1, 1)
        args.mode = saved_mode
        solvers.COARSE_TEST = forced
        line["other_operand_mode"] = {"mode": other, "launch_ms": o_ms,
                                      "ms_per_100_iters": o_solve_ms,
                                      "achieved": orf["achieved"], "peak": orf["peak"],
                                      "frac": orf["frac"]}
        set_mode(args.mode)
    if args.copy_calibration:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(x, y, a, b)
    if args.cpu_configs:
        line["cpu_baseline_other_configs"] = cpu_baseline_other_configs()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
