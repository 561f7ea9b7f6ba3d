"""Posterior moments at full size: BASELINE configs[1] (one window, 58368 rows, 22->40->1, Gaussian
likelihood sigma = 0.01, prior N(0, 0.1^2), 1000 leapfrog steps, 100 burn-in transitions with the
reference's step-size adaptation from eps0 = 0.01, 800 kept samples) run once by the oracle on the CPU and
once by the library on the GPU with the same RNG streams, then compared statistically.

Not collected by pytest (the oracle's chain is 900 000 gradient evaluations: about an hour on 8 cores);
the reduced-size counterpart that runs in the suite is test_posterior_moments_over_800_samples.

    python tests/full_size_posterior.py oracle ORACLE.npz      # CPU only, prints progress
    python tests/full_size_posterior.py gpu GPU.npz             # needs an MI355X, a few seconds
    python tests/full_size_posterior.py gpu4 GPU4.npz           # yardstick: four GPU chains on the same window
    python tests/full_size_posterior.py spread GPU4.npz         # how far chains of ONE sampler end up apart
    python tests/full_size_posterior.py compare ORACLE.npz GPU.npz [GPU4.npz]

The yardstick matters: the comparison of two chains is only a parity statement if the chain mixes within
its 800 samples.  `spread` answers that with the library's own chains: same data, same code, only the
momentum streams differ (split R-hat over four chains, and the same z statistic between two of them).
"""
import math
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

N, D0, D1, L, BURN, KEEP, SEED = 58368, 22, 40, 1000, 100, 800, 0


def run_oracle(out):
    import orc_binding as ob

    orc = ob.load()
    om = ob.Model(D0, D1, N, ob.LIK_GAUSSIAN, 0.01, 0.0, 0.1)
    oh = ob.Hmc(L, BURN, KEEP, BURN, 0.01, 0.2, 0.1, 0.01, SEED, 0)
    X, y, _ = orc.gen_window(SEED, 0, N, teacher_scale=0.1, noise_sigma=0.01)
    P = orc.num_params(D0, D1)
    T = BURN + KEEP
    samples = np.full((KEEP, P), np.nan, np.float32)
    la, acc, eps = np.empty(T, np.float32), np.empty(T, np.int32), np.empty(T, np.float32)
    w, e, t = None, 0.01, 0
    t_start = time.time()
    while t < T:
        k = min(10, T - t)
        # a chain continued from a saved state equals the tail of the whole chain (pinned in
        # tests/test_oracle_pins.py), so the run can be cut into pieces that report progress
        r = orc.run_chain_from(om, oh, X, y, w, e, t, k)
        la[t:t + k], acc[t:t + k], eps[t:t + k] = r["log_acpt"], r["accept"], r["eps"]
        filled = ~np.isnan(r["samples"][:, 0])
        samples[filled] = r["samples"][filled]
        w, e, t = r["final_w"], r["final_eps"], t + k
        print("[oracle] %d/%d transitions, %d accepted, eps %.4g, %.0f s" % (t, T, acc[:t].sum(), e,
                                                                           time.time() - t_start), flush=True)
    assert not np.isnan(samples).any()
    np.savez(out, samples=samples, log_acpt=la, accept=acc, eps=eps)


def run_gpu(out):
    import __graft_entry__ as ge

    pkg = ge.load_package()
    lib = pkg.load()
    model = lib.default_model(n=N, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=0.01, prior_scale=0.1)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=BURN, n_samples=KEEP, eps0=0.01, seed=SEED)
    s = lib.create(model, hmc, lib.default_launch(), 1, 1)  # one chain on all 256 CUs
    s.generate_window(0, teacher_scale=0.1, noise_sigma=0.01)
    s.init_chains(None)
    t0 = time.time()
    s.run(BURN + KEEP)
    print("[gpu] %d transitions in %.1f s" % (BURN + KEEP, time.time() - t0), flush=True)
    tr = s.get_traces(0)
    np.savez(out, samples=s.get_samples(0), log_acpt=tr["log_acpt"], accept=tr["accept"], eps=tr["eps"])
    s.close()


def run_gpu4(out):
    import __graft_entry__ as ge

    pkg = ge.load_package()
    lib = pkg.load()
    model = lib.default_model(n=N, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=0.01, prior_scale=0.1)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=BURN, n_samples=KEEP, eps0=0.01, seed=SEED)
    s = lib.create(model, hmc, lib.default_launch(), 1, 4)  # four chains on the window's rows
    s.generate_window(0, teacher_scale=0.1, noise_sigma=0.01)
    s.init_chains(None)
    t0 = time.time()
    s.run(BURN + KEEP)
    print("[gpu] 4 chains x %d transitions in %.1f s" % (BURN + KEEP, time.time() - t0), flush=True)
    samples = np.stack([s.get_samples(c) for c in range(4)])
    acc = np.stack([s.get_traces(c)["accept"] for c in range(4)])
    rhat, ess = lib.split_rhat_ess(samples)
    np.savez(out, samples=samples, accept=acc, rhat=rhat, ess=ess)
    s.close()


def spread(f):
    d = np.load(f)
    x = d["samples"].astype(np.float64)
    rhat, ess = d["rhat"], d["ess"]
    print("four chains of one sampler on the same window (chain ids 0..3: only the momentum and accept streams "
          "differ); accept rates over the kept samples: %s" % " ".join("%.3f" % a[BURN:].mean() for a in d["accept"]))
    print("split R-hat over the 961 weights: median %.2f, 90th percentile %.2f, max %.2f; %.1f %% above 1.1" % (
        np.median(rhat), np.percentile(rhat, 90), rhat.max(), 100 * np.mean(rhat > 1.1)))
    print("effective sample size of the 4 x 800 draws: median %.0f, min %.1f" % (np.median(ess), ess.min()))
    se = np.sqrt(batch_means_se(x[0]) ** 2 + batch_means_se(x[1]) ** 2)
    z = np.abs(x[0].mean(0) - x[1].mean(0)) / se
    ratio = x[0].std(0) / x[1].std(0)
    print("chain 0 against chain 1, the statistic of `compare`: max |z| = %.2f, %.1f %% above 2, %.1f %% above 3; "
          "std ratios min %.3f, median %.3f, max %.3f" % (z.max(), 100 * np.mean(z > 2), 100 * np.mean(z > 3),
                                                           ratio.min(), np.median(ratio), ratio.max()))


def batch_means_se(x, nb=20):
    bm = x.reshape(nb, -1, x.shape[1]).mean(1)
    return bm.std(0, ddof=1) / math.sqrt(nb)


def compare(fa, fb, fyard=None):
    a, b = np.load(fa), np.load(fb)
    sa, sb = a["samples"].astype(np.float64), b["samples"].astype(np.float64)
    first = int(np.argmax(a["accept"] != b["accept"])) if (a["accept"] != b["accept"]).any() else len(a["accept"])
    print("first transition whose decision differs: %d of %d (the first 50 must be equal: %s)" % (
        first, len(a["accept"]), "yes" if first >= 50 else "NO"))
    same_eps = int(np.argmax(a["eps"] != b["eps"])) if (a["eps"] != b["eps"]).any() else len(a["eps"])
    print("step-size traces bit-equal up to transition %d; final step sizes %.6g / %.6g" % (
        same_eps, a["eps"][-1], b["eps"][-1]))
    print("accept rate over the 900 transitions: %.3f / %.3f; over the 800 kept: %.3f / %.3f" % (
        a["accept"].mean(), b["accept"].mean(), a["accept"][BURN:].mean(), b["accept"][BURN:].mean()))
    se = np.sqrt(batch_means_se(sa) ** 2 + batch_means_se(sb) ** 2)  # Monte-Carlo error of a difference
    z = np.abs(sa.mean(0) - sb.mean(0)) / se
    print("posterior means of the %d weights: max |z| = %.2f, %.1f %% above 2, %.1f %% above 3 "
          "(z = difference / batch-means standard error of the difference, 20 batches of 40 samples)" % (
              z.size, z.max(), 100 * np.mean(z > 2), 100 * np.mean(z > 3)))
    ratio = sa.std(0) / sb.std(0)
    print("posterior std ratios: min %.3f, median %.3f, max %.3f" % (ratio.min(), np.median(ratio), ratio.max()))
    print("largest |mean| %.3f, mean posterior std %.4f, mean standard error of a difference %.4f" % (
        np.abs(sa.mean(0)).max(), sa.std(0).mean(), se.mean()))
    ok = first >= 50 and z.max() < 5.0 and np.mean(z > 3.0) < 0.02 and 0.5 < ratio.min() and ratio.max() < 2.0
    print("against the bounds of a chain that mixes (max |z| < 5, under 2 %% above 3, std ratios in [0.5, 2]): %s" % (
        "within Monte-Carlo error" if ok else "OUTSIDE"))
    if fyard is None:
        return 0 if ok else 1
    # the yardstick: two chains of one sampler (same data, same code, different momentum streams)
    x = np.load(fyard)["samples"].astype(np.float64)
    zy = np.abs(x[0].mean(0) - x[1].mean(0)) / np.sqrt(batch_means_se(x[0]) ** 2 + batch_means_se(x[1]) ** 2)
    print("the same statistic between two chains of ONE sampler: max |z| = %.2f, %.1f %% above 3" % (
        zy.max(), 100 * np.mean(zy > 3)))
    same = first >= 50 and z.max() <= 1.5 * zy.max() and np.mean(z > 3) <= np.mean(zy > 3) + 0.1
    print("result: the two implementations are %s than two chains of one implementation" % (
        "no further apart" if same else "FURTHER APART"))
    return 0 if same else 1


if __name__ == "__main__":
    if len(sys.argv) == 3 and sys.argv[1] == "oracle":
        run_oracle(sys.argv[2])
    elif len(sys.argv) == 3 and sys.argv[1] == "gpu":
        run_gpu(sys.argv[2])
    elif len(sys.argv) == 3 and sys.argv[1] == "gpu4":
        run_gpu4(sys.argv[2])
    elif len(sys.argv) == 3 and sys.argv[1] == "spread":
        spread(sys.argv[2])
    elif len(sys.argv) in (4, 5) and sys.argv[1] == "compare":
        sys.exit(compare(*sys.argv[2:]))
    else:
        print(__doc__)
        sys.exit(2)
