#!/usr/bin/env python3
"""Benchmark of the HMC hot path on one MI355X.

Workload (BASELINE.json configs[2], the configuration the metric is quoted on): 200 independent windows
of the 22->40->1 Bayesian MLP, full batch of 58368 rows each (features ~ N(0,1), teacher-MLP targets +
N(0, 0.01^2) noise, Gaussian likelihood, Gaussian weight prior), one chain per window, HMC with 1000
leapfrog steps per transition, all 200 windows resident in HBM (1.07 GB).  A "step" is one HMC transition
(momentum resampling, 1000 fused leapfrog gradient evaluations, log accept ratio, Metropolis decision,
sample store) of every one of the 200 windows: the chains take turns, five transitions at a time, on
launches of 64 chains at 4 workgroups per chain (of the rows of 64 windows, 344 MB, the 256 MB memory-side
cache serves most from one leapfrog step to the next, because a wave walks its tiles back and forth) or of 128
chains at 2, whichever the library measures to be faster in the warm-up call; what does not fill such a launch
runs as 32 chains at 8, 16 at 16, ... workgroups per chain, always over all 256 compute units.  The warm-up transitions
are the burn-in (nothing stored), the timed ones store their samples.  The metric is leapfrog gradient
evaluations per second; the minutes for 200 windows x (100 burn-in + 800 samples) are 900 steps plus the
bootstrap evaluation, and --full runs that whole job.

Prints ONE JSON line.  Inputs are resident in HBM before the timed region starts.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_ROWS, D0, D1 = 58368, 22, 40
FLOP_PER_EVAL = 4 * N_ROWS * D1 * (D0 + 1)  # 214,794,240: both layers, forward + weight gradients
# --shape wide: BASELINE.json configs[4], 64->128->1 on 4 x 58368 rows, 4 chains per window
WIDE_ROWS, WIDE_D0, WIDE_D1, WIDE_CHAINS = 4 * 58368, 64, 128, 4
PEAK_TFLOPS = 157.3                         # MI355X dense FP32 matrix peak (v_mfma_f32_16x16x4_f32)
EVALS_200x800 = 200 * (900 * 1000 + 1)      # 200 windows x ((100 + 800) transitions x 1000 steps + bootstrap)
EVALS_200x1600 = 200 * (1700 * 1000 + 1)
# HBM-side bytes per gradient evaluation of the trajectory kernels, measured with rocprofv3 FETCH_SIZE
# and WRITE_SIZE scaled by a 1 GiB copy kernel: written by mcmc-bnn-example_amd/profile_summary.py
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(kernel_key):
    """bytes per gradient evaluation of `kernel_key` from profiles/traffic.json, or None"""
    try:
        with open(TRAFFIC_JSON) as f:
            return float(json.load(f)[kernel_key]["bytes_per_grad_eval"])
    except (OSError, KeyError, ValueError, TypeError):
        return None


def batch_plan(n_chains, resident_wgs, cus_per_chain, wide, max_chains):
    """[(chains, workgroups per chain)] of the launches that cover n_chains, as the library lays them out:
    a fixed group size when one is configured (the 64->128->1 default is 4), otherwise the largest
    power-of-two number of chains that is left and fits (max_chains: what the library says fits, which
    may keep a launch's rows within 1.4 times the memory-side cache), spread over the whole device; a batch that
    leaves compute units idle gets its groups doubled while they still fit."""
    def widen(g, b):
        while g * 2 * b <= resident_wgs and g * 2 <= 256:
            g *= 2
        return g
    fixed = cus_per_chain or (4 if wide else 0)
    out, left = [], n_chains
    while left > 0:
        if fixed:
            b = min(left, max(1, resident_wgs // fixed))
            g = fixed if cus_per_chain else widen(fixed, b)
        else:
            b = 1
            while b * 2 <= min(left, resident_wgs, max_chains):
                b *= 2
            g = widen(1, b)
        out.append((b, g))
        left -= b
    return out


def cpu_baseline(seconds, n_rows=N_ROWS, d0=D0, d1=D1):
    """The CPU oracle (a port of the reference math), timed on this host's cores on one window."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import orc_binding as ob

    orc = ob.load()
    X, y, _ = orc.gen_window(0, 0, n_rows, d0=d0, d1=d1)
    m = ob.gauss_model(n=n_rows, d0=d0, d1=d1)
    threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
    threads = max(1, min(threads, os.cpu_count() or 1))
    rate, used, done = orc.bench_grad_evals(m, X, y, threads, seconds)
    return {"value": rate, "unit": "grad-evals/s", "cores": used, "kind": "port",
            "sample": "%d leapfrog gradient evaluations of one %d-row window in %.0f s, one chain per "
                      "thread" % (done, n_rows, seconds),
            "extrapolated_minutes_200x800": EVALS_200x800 / rate / 60.0 if d0 == D0 else None}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20, help="timed HMC transitions of the batch")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layer", choices=["mfma", "ffma"], default="mfma")
    ap.add_argument("--cus-per-chain", type=int, default=0)
    ap.add_argument("--wgs-per-cu", type=int, default=0)
    ap.add_argument("--threads", type=int, default=0)
    ap.add_argument("--pipeline", type=int, default=0)
    ap.add_argument("--windows", type=int, default=0,
                    help="0 = 200 (the configuration the metric is quoted on); --shape wide: as many as are "
                         "co-resident")
    ap.add_argument("--leapfrog", type=int, default=1000)
    ap.add_argument("--transitions-per-launch", type=int, default=5)
    ap.add_argument("--eps0", type=float, default=2e-5,
                    help="leapfrog step size of the timed transitions: what the adaptation reaches on this "
                         "posterior; --full starts from the reference's 0.01 and adapts")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="0 skips the CPU baseline")
    ap.add_argument("--shape", choices=["base", "wide"], default="base",
                    help="base = configs[2] (22->40->1, the metric's configuration); wide = configs[4] "
                         "(64->128->1, 233472 rows, 4 chains per window)")
    ap.add_argument("--full", action="store_true",
                    help="run the whole 200 windows x (100 + 800) transitions job from the all-zero start with "
                         "the reference's adaptation and time all of it")
    ap.add_argument("--lik", choices=["gaussian", "student_t"], default="gaussian",
                    help="gaussian = the benchmark configurations (sigma 0.01, prior N(0, 0.1^2)); student_t = the "
                         "reference's own model constants (Student-t scale 100, 2.2 degrees of freedom, prior scale "
                         "200) on the same synthetic data")
    ap.add_argument("--samples", type=int, default=800, choices=[800, 1600],
                    help="--full only: kept samples per window (800 = configs[2], 1600 = configs[3])")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU (windows are independent: more GPUs would only run more windows "
              "side by side); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import __graft_entry__ as ge

    pkg = ge.load_package()
    lib = pkg.load()
    rc, n_dev, cus, arch = lib.device_info()
    if rc != 0:
        print("no MI355X visible: %s" % lib.c.bnnhmc_last_error().decode(), file=sys.stderr)
        sys.exit(1)

    layer = pkg.LAYER_MFMA if args.layer == "mfma" else pkg.LAYER_FFMA
    launch = lib.default_launch(layer=layer, transitions_per_launch=args.transitions_per_launch)
    if args.cus_per_chain:
        launch.cus_per_chain = args.cus_per_chain
    if args.wgs_per_cu:
        launch.wgs_per_cu = args.wgs_per_cu
    if args.threads:
        launch.threads = args.threads
    if args.pipeline:
        launch.pipeline = args.pipeline
    wide = args.shape == "wide"
    if wide and args.full:
        print("--full is the 22->40->1 job; it is not defined for --shape wide", file=sys.stderr)
        sys.exit(2)
    n_rows, d0, d1, cpw = (WIDE_ROWS, WIDE_D0, WIDE_D1, WIDE_CHAINS) if wide else (N_ROWS, D0, D1, 1)
    flop_per_eval = 4 * n_rows * d1 * (d0 + 1)
    wgs_per_cu = 1 if wide or layer != pkg.LAYER_MFMA else launch.wgs_per_cu
    resident_wgs = cus * wgs_per_cu
    n_windows = args.windows or (max(1, resident_wgs // 4 // cpw) if wide else 200)
    n_chains = n_windows * cpw

    student = args.lik == "student_t"
    if student:
        model = lib.default_model(d0=d0, d1=d1, n=n_rows)  # global_params.h:39-48
        if args.eps0 == 2e-5:
            args.eps0 = 0.027  # what the adaptation reaches with this model on this data
    else:
        model = lib.default_model(d0=d0, d1=d1, n=n_rows, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=0.01,
                                  prior_scale=0.1)
    if args.full:
        burn, keep, adapt = 100, args.samples, 100
    else:  # warm-up = burn-in (nothing stored), timed transitions store their samples; no adaptation
        burn, keep, adapt = args.warmup, args.steps, 0
    hmc = lib.default_hmc(leapfrog_steps=args.leapfrog, burn_in=burn, n_samples=keep, adapt_steps=adapt, seed=0)
    if not args.full:
        hmc.eps0 = args.eps0
    s = lib.create(model, hmc, launch, n_windows, cpw)
    teachers = []
    t_gen = time.perf_counter()
    for w in range(n_windows):
        teachers.append(s.generate_window(w, teacher_scale=0.1, noise_sigma=0.01))  # untimed, like the reference's load
    print("[bench] %d windows generated and uploaded in %.1f s" % (n_windows, time.perf_counter() - t_gen),
          file=sys.stderr, flush=True)

    if args.full:
        # the reference's timed region: bootstrap + every transition (main.h:187-293)
        t0 = time.perf_counter()
        s.init_chains(None)
        steps, warm, done = burn + keep, 0, 0
        while done < steps:
            # long calls: the chains take turns on launches of the widest batch, and only what is left at
            # the end of a call runs in narrower ones
            k = min(100, steps - done)
            s.run(k)
            done += k
            print("[bench] %d/%d transitions of %d windows, %.0f s" % (
                done, steps, n_windows, time.perf_counter() - t0), file=sys.stderr, flush=True)
        wall = time.perf_counter() - t0
        tm0 = dict(kernel_ms=0.0, launches=0)
    else:
        # every chain starts at its window's teacher weights (the region the burn-in of the whole job ends
        # in) with the adapted step size, so that the timed transitions accept at the rate the job's do
        s.init_chains(None)
        for c in range(n_chains):
            s.set_chain_state(c, teachers[c // cpw], args.eps0, 0, 0)
        steps, warm = args.steps, args.warmup
        if warm:
            s.run(warm)
        tm0 = s.timing()
        t0 = time.perf_counter()
        s.run(steps)  # synchronous at return: the stream is drained
        wall = time.perf_counter() - t0
    tm1 = s.timing()
    # the batch the library ended up with (where two shapes compete it has timed a launch of each)
    batching, trial = s.batching(), s.batch_trial_rates()
    plan = batch_plan(n_chains, resident_wgs, launch.cus_per_chain, wide, batching[0])
    assert plan[0] == batching, (plan[0], batching)
    resident = plan[0][0]                                   # chains in flight in a full launch
    states = [s.get_chain_state(c) for c in range(n_chains)]
    stored = s.get_samples(0).shape[0]
    s.close()
    n_acc = sum(st["n_accepted"] for st in states)
    n_done = sum(st["transitions_done"] for st in states)

    evals = n_chains * steps * args.leapfrog + (n_chains if args.full else 0)
    value = evals / wall
    ms_per_step = wall * 1e3 / steps
    # dominant kernel: the trajectory kernel.  Average launch duration from HIP events recorded on the
    # sampler's stream around the launches of the timed region.
    dev_ms = tm1["kernel_ms"] - tm0["kernel_ms"]
    launches = tm1["launches"] - tm0["launches"]
    ms_per_launch = dev_ms / max(1, launches)
    evals_per_launch = (n_chains * steps * args.leapfrog) / max(1, launches)
    achieved = flop_per_eval * evals_per_launch / (ms_per_launch * 1e-3) / 1e12
    kernel_key = "hmc_kernel_wide_64x128" if wide else "hmc_kernel_%s_22x40" % args.layer
    bytes_per_eval = measured_traffic(kernel_key)

    out = {
        "metric": "leapfrog grad-evals/sec (minutes for 200 windows x 800 samples derived), 1 MI355X",
        "value": value,
        "unit": "grad-evals/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warm,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[%s]: %d independent windows x %d chain(s), all resident in HBM (%d chains in "
                        "flight per launch), %d->%d->1 BNN, %dx%d features ~N(0,1), teacher-MLP targets + "
                        "N(0,0.01^2), %s, %d leapfrog steps per transition; one step "
                        "= one transition of every window, samples stored in the timed region" % (
                            "4" if wide else ("3" if args.full and keep == 1600 else "2"), n_windows, cpw,
                            min(n_chains, resident), d0, d1, n_rows, d0,
                            "Student-t likelihood (scale 100, 2.2 degrees of freedom) and prior scale 200 as in the "
                            "reference" if student else "Gaussian likelihood and prior", args.leapfrog),
            "layer": args.layer, "wgs_per_cu": wgs_per_cu,
            "launches_chains_x_workgroups_per_chain": (
                "%d x %d, the %d chains taking turns in quanta of %d transitions; what does not fill a launch runs "
                "in the largest batches that fit (%s)" % (
                    plan[0][0], plan[0][1], n_chains, args.transitions_per_launch,
                    ", ".join("%d x %d" % bg for bg in sorted(set(plan[1:]), reverse=True)))
                if not wide and not launch.cus_per_chain and len(plan) > 1
                else ", ".join("%d x %d" % bg for bg in plan)),
            "batch_shape_trial": None if trial[0] <= 0 else (
                "the library timed one launch of each shape at the start of the %s: rows of a launch within 1.4 "
                "times the memory-side cache %.0f evals/s, as many chains as fit the device %.0f evals/s" % (
                    "last call of the job" if args.full else "warm-up call", trial[0], trial[1])),
            "workgroups_last_launch": tm1["workgroups"], "compute_units": cus,
            "transitions_per_launch": args.transitions_per_launch,
            "eps0": float(hmc.eps0), "adapt_steps": int(hmc.adapt_steps),
            "samples_stored_per_chain": int(stored),
        },
        # 100 burn-in + 800 kept transitions of all 200 windows, plus the bootstrap evaluation (one
        # gradient evaluation per window: 1/1000 of a step)
        "minutes_200x800": None if wide or n_windows != 200 else (
            wall / 60.0 if args.full and keep == 800 else (900 + 0.001) * ms_per_step / 6e4),
        "minutes_200x800_kind": "not defined for this workload" if wide or n_windows != 200 else (
            "measured: the whole job was run" if args.full and keep == 800 else
            "900 x the measured time of one transition of all 200 windows"),
        "minutes_200x1600": None if wide or n_windows != 200 else (
            wall / 60.0 if args.full and keep == 1600 else (1700 + 0.001) * ms_per_step / 6e4),
        "minutes_200x1600_kind": "not defined for this workload" if wide or n_windows != 200 else (
            "measured: the whole job was run" if args.full and keep == 1600 else
            "1700 x the measured time of one transition of all 200 windows"),
        "reference_minutes_200x800_1xA100_tf32": 42,
        "accept_rate": n_acc / max(1, n_done),
        "eps_chain0": states[0]["eps"],
        "roofline": {
            "bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / PEAK_TFLOPS,
            "traffic": None if bytes_per_eval is None else bytes_per_eval * evals_per_launch,
            "traffic_unit": "HBM bytes per launch: rocprofv3 FETCH_SIZE + WRITE_SIZE per gradient evaluation "
                            "(profiles/traffic.json) x the evaluations of an average launch",
            # compulsory bytes: a chain's rows (X and y) once per trajectory
            "algorithmic_bytes_per_launch": (n_rows * (d0 + 1) * 4) * evals_per_launch / args.leapfrog,
            "kernel": "hmc_kernel_wide" if wide else "hmc_kernel", "launches": launches,
            "ms_per_launch": ms_per_launch, "flop_per_grad_eval": flop_per_eval,
            "grad_evals_per_launch": evals_per_launch,
        },
    }
    if args.cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline(args.cpu_seconds, n_rows, d0, d1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
