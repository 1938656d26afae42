"""Per-operation timings at the benchmark shapes: ``python -m flash_sinkhorn_amd.op_timings [c1 c2 c3 c4 c5]``.

Prints one JSON line per shape with the average launch time (HIP events on the current
stream) and the algorithmic rate of every C-ABI operation: symmetric step (4nmd flop; alone, and
as a solver loop runs it: on planes converted once, where a step whose sums have settled takes
both sides from one sweep over the logits and ``one_sweep`` says whether the timed steps did;
likewise a step of the two self problems x-with-x and y-with-y, 2(n^2 + m^2)d flop),
one LSE half-update (2nmd), gradient of one side (4nmd), plan-vector (2nmd), plan-matrix
(4nmd), mat5 (6nmd) and the hard c-transform (2nmd); at c3 also the gradient after a solve on clustered clouds,
with and without the keys the solve carried; then end-to-end wall times of the five configurations
through the public API (solver loops, autograd, CG included).

``python -m flash_sinkhorn_amd.op_timings clocks`` instead runs four operations in a loop for a
few seconds each and prints the shader clock that ``rocm-smi`` reports meanwhile (the clock the
chip sustains under that load, against the one it reaches for a plain device copy).
"""
from __future__ import annotations

import json
import sys
import time

import torch

from flash_sinkhorn_amd import SamplesLoss, _lib, c_transform_fwd
from flash_sinkhorn_amd.kernels import sinkhorn_flashstyle_alternating
from flash_sinkhorn_amd.kernels.apply_flash import (apply_plan_mat_flashstyle,
                                                    apply_plan_vec_flashstyle)
from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid
from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (_self_pair_steps_raw,
                                                                     _symmetric_step_raw,
                                                                     flashsinkhorn_lse_fused)
from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
    sinkhorn_geomloss_online_grad_sqeuclid)

SHAPES = {"c1": (2000, 2000, 3, 0.01), "c2": (10000, 10000, 64, 0.01),
          "c3": (50000, 50000, 64, 0.01), "c4": (20000, 30000, 128, 0.0025),
          "c5": (8192, 8192, 1536, 0.25)}


def _avg_ms(fn, reps=5):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def _wall_ms(fn, reps=4, warm=3):
    for _ in range(warm):  # small solves run eagerly once, capture a graph once, then replay
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / reps


def kernel_timings(name):
    n, m, d, eps = SHAPES[name]
    gen = torch.Generator(device="cuda").manual_seed(0)
    sc = 2.0 / d ** 0.5
    X = torch.randn(n, d, device="cuda", generator=gen) * sc
    Y = torch.randn(m, d, device="cuda", generator=gen) * sc
    A = torch.full((n,), 1.0 / n, device="cuda")
    B = torch.full((m,), 1.0 / m, device="cuda")
    la, lb = A.log(), B.log()
    al, be = (X * X).sum(1), (Y * Y).sum(1)
    fh, gh = -al, -be
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    for _ in range(3):  # a few iterations so that the plan is not degenerate
        fh, gh = _symmetric_step_raw(X, Y, fh, gh, la, lb, eps, **kw)
    f, g = fh + al, gh + be
    v = torch.randn(m, device="cuda", generator=gen)
    V = torch.randn(m, d, device="cuda", generator=gen)
    Am = torch.randn(n, d, device="cuda", generator=gen)
    fo, go = f + eps * la, g + eps * lb
    nmd = float(n) * m * d
    ops = {
        "symmetric_step": (4, lambda: _symmetric_step_raw(X, Y, fh, gh, la, lb, eps, **kw)),
        "lse_half": (2, lambda: flashsinkhorn_lse_fused(X, Y, gh, lb, eps, allow_tf32=False)),
        "grad_x": (4, lambda: sinkhorn_geomloss_online_grad_sqeuclid(
            X, Y, A, B, f, g, eps=eps, allow_tf32=False, compute_grad_y=False)),
        "apply_vec": (2, lambda: apply_plan_vec_flashstyle(X, Y, fh, gh, la, lb, v, eps=eps,
                                                           axis=1)),
        "apply_mat": (4, lambda: apply_plan_mat_flashstyle(X, Y, fh, gh, la, lb, V, eps=eps,
                                                           axis=1)),
        "mat5": (6, lambda: mat5_sqeuclid(X, Y, fo, go, Am, eps=eps)),
        "c_transform": (2, lambda: c_transform_fwd(X, Y, g, allow_tf32=False)),
    }
    out = {"shape": name, "n": n, "m": m, "d": d}
    for op, (k, fn) in ops.items():
        ms = _avg_ms(fn)
        out[op] = {"ms": round(ms, 4), "algorithmic_TFLOPs": round(k * nmd / ms / 1e9, 1)}
    # the step inside a solver loop: planes converted once, a few more steps so that it settles
    prep = _lib.PreparedOperands(X, Y, _lib.flags(True, False))
    f2, g2 = fh, gh
    for _ in range(6):
        f2, g2 = _symmetric_step_raw(X, Y, f2, g2, la, lb, eps, prepared=prep, **kw)
    ms = _avg_ms(lambda: _symmetric_step_raw(X, Y, f2, g2, la, lb, eps, prepared=prep, **kw))
    out["symmetric_step_in_a_loop"] = {"ms": round(ms, 4), "algorithmic_TFLOPs": round(4 * nmd / ms / 1e9, 1),
                                       "one_sweep": bool(prep.variant_state()["sweep_next"])}
    # a step of the two self problems of a debiased loss (x with x, y with y), in a loop
    prep2 = _lib.PreparedOperands(X, Y, _lib.flags(True, False), self_pair=True)
    skw = dict(cost_scale=1.0, allow_tf32=False, prepared=prep2)
    sx, sy = _self_pair_steps_raw(X, Y, -al, -be, la, lb, [(eps, eps, 1.0, 1.0, 1.0)] + [(eps, eps, 0.5, 1.0, 1.0)] * 7, **skw)
    ms = _avg_ms(lambda: _self_pair_steps_raw(X, Y, sx, sy, la, lb, [(eps, eps, 0.5, 1.0, 1.0)] * 10, **skw), reps=2) / 10
    out["self_pair_step_in_a_loop"] = {"ms": round(ms, 4),
                                       "algorithmic_TFLOPs": round(2 * (float(n) * n + float(m) * m) * d / ms / 1e9, 1),
                                       "one_sweep": bool(prep2.variant_state()["sweep_next"])}
    return out


def end_to_end(name):
    n, m, d, eps = SHAPES[name]
    gen = torch.Generator(device="cuda").manual_seed(1)
    X = torch.randn(n, d, device="cuda", generator=gen)
    Y = torch.randn(m, d, device="cuda", generator=gen)
    if name == "c5":
        X, Y = X / d ** 0.5, Y / d ** 0.5
    out = {"config": name}
    if name in ("c1", "c2", "c3", "c5"):
        kw = dict(blur=eps ** 0.5, use_epsilon_scaling=False, eps=eps,
                  n_iters=50 if name == "c5" else 100, allow_tf32=False,
                  half_cost=(name == "c1"), debias=(name != "c3"))
        Xg = X.clone().requires_grad_(True)

        def loss_and_grad():
            loss = SamplesLoss("sinkhorn", **kw)(Xg, Y)
            return torch.autograd.grad(loss, Xg)
        out["loss_and_grad_x_ms"] = round(_wall_ms(loss_and_grad), 2)
        if name in ("c2", "c3"):  # what a user who passes no options gets (eps-scaling, debiased)
            out["samples_loss_defaults_ms"] = round(_wall_ms(lambda: SamplesLoss()(X, Y)), 2)
        if name == "c5":
            Vv = torch.randn(n, d, device="cuda", generator=gen)
            kw2 = dict(kw, debias=False, hvp_max_cg_iter=20)

            def hvp():
                loss = SamplesLoss("sinkhorn", **kw2)(Xg, Y)
                (g1,) = torch.autograd.grad(loss, Xg, create_graph=True)
                return torch.autograd.grad((g1 * Vv).sum(), Xg)
            out["loss_grad_hvp_ms"] = round(_wall_ms(hvp), 2)
    else:
        A = torch.rand(n, device="cuda", generator=gen)
        B = torch.rand(m, device="cuda", generator=gen)
        A, B = A / A.sum(), 1.3 * B / B.sum()
        out["alternating_10_iters_ms"] = round(_wall_ms(lambda: sinkhorn_flashstyle_alternating(
            X, Y, A, B, eps=eps, n_iters=10, reach=1.0, threshold=1e-3, check_every=10,
            allow_tf32=False)), 2)
    return out


def gradient_after_solve(name):
    """Both-sides gradient at the potentials of a 100-iteration fixed-eps solve on clustered
    clouds (8-component Gaussian mixtures, a peaked plan): without hints, and with the keys the
    solve carried (what the loss's backward passes to fs_grad_seeded)."""
    import numpy as np

    from flash_sinkhorn_amd import sinkhorn_solvers as solvers
    n, m, d, eps = SHAPES[name]
    rng = np.random.default_rng(3)

    def cloud(rows):
        centres = rng.standard_normal((8, d)).astype(np.float32) * 0.6
        pts = centres[rng.integers(0, 8, rows)] + 0.25 * rng.standard_normal((rows, d)).astype(np.float32)
        return torch.from_numpy(pts.astype(np.float32)).cuda()

    X, Y = cloud(n), cloud(m)
    A = torch.full((n,), 1.0 / n, device="cuda")
    B = torch.full((m,), 1.0 / m, device="cuda")
    info = {}
    f, g = solvers.sinkhorn_flashstyle_symmetric(X, Y, A, B, use_epsilon_scaling=False, eps=eps,
                                                 n_iters=100, allow_tf32=False, solve_info=info)[:2]
    prep = info.get("prepared")
    keys = None
    if prep is not None and prep.best_keys(0) is not None:
        keys = (prep.best_keys(0).clone(), prep.best_keys(1).clone())
    out = {"shape": name, "workload": "gradient of both sides after a 100-iteration solve, "
                                      "8-component Gaussian mixtures"}
    for label, k in (("ms_without_hints", None), ("ms_with_carried_keys", keys)):
        if label == "ms_with_carried_keys" and k is None:
            continue
        out[label] = round(_avg_ms(lambda: sinkhorn_geomloss_online_grad_sqeuclid(
            X, Y, A, B, f, g, eps=eps, allow_tf32=False, _seed_keys=k), reps=10), 4)
    return out


def clocks_under_load(seconds=4.0):
    """Shader clock (rocm-smi, sampled every 0.15 s from a second thread) while one operation
    runs back to back: the large-d plan-matrix and plan-vector products, the two-sided
    symmetric step at the benchmark size, and a 1 GiB device copy for comparison."""
    import re
    import subprocess
    import threading

    def sclk():
        try:
            out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True,
                                 timeout=10).stdout
            hit = re.search(r"sclk clock level[^(]*\((\d+)Mhz\)", out)
            return int(hit.group(1)) if hit else None
        except (OSError, subprocess.SubprocessError):
            return None

    def measure(label, fn):
        fn()
        torch.cuda.synchronize()
        stop, samples = [False], []

        def poll():
            while not stop[0]:
                samples.append(sclk())
                time.sleep(0.15)
        th = threading.Thread(target=poll)
        th.start()
        t0, launches = time.perf_counter(), 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            launches += 20
        dt = time.perf_counter() - t0
        stop[0] = True
        th.join()
        got = sorted(v for v in samples[2:-1] if v is not None)
        return {"operation": label, "ms_per_launch": round(dt / launches * 1e3, 3),
                "sclk_mhz_min_median_max": [got[0], got[len(got) // 2], got[-1]] if got else None,
                "samples": len(got)}

    gen = torch.Generator(device="cuda").manual_seed(0)
    n, m, d, eps = SHAPES["c5"]
    X = torch.randn(n, d, device="cuda", generator=gen) * (2.0 / d ** 0.5)
    Y = torch.randn(m, d, device="cuda", generator=gen) * (2.0 / d ** 0.5)
    la = torch.full((n,), 1.0 / n, device="cuda").log()
    lb = torch.full((m,), 1.0 / m, device="cuda").log()
    f, g = -(X * X).sum(1), -(Y * Y).sum(1)
    V = torch.randn(m, d, device="cuda", generator=gen)
    v = torch.randn(m, device="cuda", generator=gen)
    out = [measure("c5 plan-matrix product (plan_gemm_kernel)", lambda: apply_plan_mat_flashstyle(
        X, Y, f, g, la, lb, V, eps=eps, axis=1, allow_tf32=False))]
    out.append(measure("c5 plan-vector product (lse_gemm_kernel)", lambda: apply_plan_vec_flashstyle(
        X, Y, f, g, la, lb, v, eps=eps, axis=1, allow_tf32=False)))
    n, m, d, eps = SHAPES["c3"]
    X = torch.randn(n, d, device="cuda", generator=gen) * (2.0 / d ** 0.5)
    Y = torch.randn(m, d, device="cuda", generator=gen) * (2.0 / d ** 0.5)
    la = torch.full((n,), 1.0 / n, device="cuda").log()
    lb = torch.full((m,), 1.0 / m, device="cuda").log()
    fh, gh = -(X * X).sum(1), -(Y * Y).sum(1)
    kw = dict(cost_scale=1.0, alpha=0.5, damping_f=1.0, damping_g=1.0, allow_tf32=False)
    out.append(measure("c3 symmetric step alone (two-sided lse2_kernel, planes converted in the call)",
                       lambda: _symmetric_step_raw(X, Y, fh, gh, la, lb, eps, **kw)))
    src = torch.empty(1 << 28, device="cuda")
    dst = torch.empty_like(src)
    out.append(measure("1 GiB device copy", lambda: dst.copy_(src)))
    return out


def main(argv):
    if "clocks" in argv:
        for line in clocks_under_load():
            print(json.dumps(line), flush=True)
        return
    names = [a for a in argv if a in SHAPES] or list(SHAPES)
    for name in names:
        print(json.dumps(kernel_timings(name)), flush=True)
    for name in names:
        if name == "c3":
            print(json.dumps(gradient_after_solve(name)), flush=True)
    for name in names:
        print(json.dumps(end_to_end(name)), flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
