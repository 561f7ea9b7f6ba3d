"""GPU tests of the two seams a maintainer of the reference would use: the operator header
include/mcmc_step_hip.h (compiled by the host compiler into mcmc-bnn-example_amd/shim_check, which walks
the start of the reference's main loop through it) and the host driver's --data route (the reference's
text format, its x0.001 feature scaling); plus properties of the ABI that callers rely on: results that do
not depend on how a job is cut into calls when the group size is fixed, bounded waits in the exchange by
slices, and the step operator's failure record staying until it is read."""
import os
import subprocess
import sys

import numpy as np
import pytest

import orc_binding as ob
from hipmem import DevBuf

pytestmark = pytest.mark.gpu

D0, D1, P = 22, 40, 961


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


# ------------------------------------------------------------------------------------------------
# include/mcmc_step_hip.h: the reference's operator interface on top of the C ABI
# ------------------------------------------------------------------------------------------------
def test_operator_header_walks_the_start_of_the_reference_main_loop(pkg, lib, orc):
    """shim_check follows main.h:117-232 with the reference's buffer rotation (Network::do_swap) around
    mcmc_step<T, 1> (bootstrap) and mcmc_step<T, 40> (one trajectory at the reference's model constants,
    58368 rows): every number it prints is compared with the oracle run on the same seeded inputs."""
    exe = os.path.join(pkg.PKG_DIR, "shim_check")
    assert os.path.exists(exe), "shim_check not built (make -C mcmc-bnn-example_amd)"
    seed, n, L, eps = 3, 58368, 40, np.float32(0.01)
    r = subprocess.run([exe, str(seed)], capture_output=True, text=True, timeout=120)
    say(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    out = {}
    for line in r.stdout.splitlines():
        tok = line.split()
        if tok and tok[0] in ("log_acpt", "w_next", "grad_cur"):
            out[tok[0]] = np.array([float(v) for v in tok[1:]])
        elif tok[:1] == ["bootstrap"] or tok[:1] == ["proposal"]:
            out[tok[0]] = (float(tok[2]), float(tok[4]))
        elif tok[:1] == ["Using"]:
            out["banner"] = line
    # main.h:121-125's banner, with this operator's constants: 2 tiles of 16 rows per wavefront, 256
    # workgroups of 8 wavefronts
    assert out["banner"].startswith("Using 32 rows/warp -> 256 blocks with 256 rows / block. Using ")
    om = ob.ref_model(n)
    X, y, _ = orc.gen_window(seed, 0, n, teacher_scale=0.3, noise_sigma=5.0)
    w0 = np.zeros(P, np.float32)
    ell0, prior0, g0, _ = orc.eval_f32(om, X, y, w0)
    m0 = orc.momentum(1, 0, 0, P)                     # SEED_INIT = 1, chain 0, transition 0
    w1, m1, g1, loss1 = orc.mcmc_step(om, X, y, w0, m0, g0, eps, L)
    la = orc.log_acpt(np.concatenate([ell0, prior0]), loss1, m0, m1, g1, eps)
    b1, b2 = out["bootstrap"]
    assert b1 == pytest.approx(float(ell0.astype(np.float64).sum()), rel=1e-6)
    assert b2 == pytest.approx(float(prior0.astype(np.float64).sum()), rel=1e-6)
    p1, p2 = out["proposal"]
    assert p1 == pytest.approx(float(loss1[:n].astype(np.float64).sum()), rel=1e-6)
    assert p2 == pytest.approx(float(loss1[n:].astype(np.float64).sum()), rel=1e-6)
    idx = np.arange(0, P, 120)
    gscale = float(np.abs(g1).max())
    assert np.abs(out["grad_cur"] - g1[idx]).max() <= 1e-5 * (L // 4) * gscale
    assert np.abs(out["w_next"] - w1[idx]).max() <= 1e-6 * L * max(1.0, float(np.abs(w1).max()))
    # the ratio is a sum of 58368 differences of per-row terms of size 5.6, each known to one FP32 ulp
    say("log accept ratio: header %.6g oracle %.6g" % (out["log_acpt"][0], la))
    assert abs(out["log_acpt"][0] - la) <= 2e-4 + 1e-5 * abs(la)


# ------------------------------------------------------------------------------------------------
# bnn_hmc_main --data: the reference's text file, features scaled by 0.001 (io.h:43-86, main.h:158-164)
# ------------------------------------------------------------------------------------------------
def test_host_driver_reads_the_reference_text_format(pkg, lib, orc, tmp_path):
    exe = os.path.join(pkg.PKG_DIR, "bnn_hmc_main")
    assert os.path.exists(exe), "driver not built"
    n, L, burn, keep, seed = 2000, 20, 4, 6, 11
    rng = np.random.default_rng(5)
    # 149 columns: two that are skipped, the label, 22 features of order 1000 (the file holds unscaled
    # features), 124 columns that are ignored; written with 9 significant digits so that strtof returns
    # these very floats
    feats = (rng.normal(0, 1000.0, (n, D0))).astype(np.float32)
    teacher = (0.3 * rng.normal(0, 1, P)).astype(np.float32)
    xs = feats * np.float32(0.001)
    h = np.tanh(xs @ teacher[:D0 * D1].reshape(D0, D1) + teacher[D0 * D1:D0 * D1 + D1])
    labels = (h @ teacher[D0 * D1 + D1:D0 * D1 + 2 * D1] + teacher[-1] + rng.normal(0, 5.0, n)).astype(np.float32)
    path = tmp_path / "returns_and_features_for_mcmc.txt"
    with open(path, "w") as f:
        f.write(" ".join("c%d" % j for j in range(149)) + "\n")
        for i in range(n):
            row = ["2020-01-%02d" % (i % 28 + 1), "ID%d" % i, "%.9g" % labels[i]]
            row += ["%.9g" % v for v in feats[i]]
            row += ["%.3f" % v for v in rng.normal(0, 1, 149 - 3 - D0)]
            f.write(" ".join(row) + "\n")
    dump = tmp_path / "chain.npy"
    r = subprocess.run([exe, "--data", str(path), "--rows", str(n), "--samples", str(keep), "--burn-in", str(burn),
                        "--leapfrog", str(L), "--seed", str(seed), "--dump", str(dump)], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "Dataset read successfully" in r.stdout and "Data: Shape: %d x 22" % n in r.stdout
    data = np.load(dump, allow_pickle=False)
    assert data.shape == (1, keep, P) and np.all(np.isfinite(data))
    # the same rows, scaled as main.h:162-164 does (one FP32 multiplication), through the library directly
    X = (feats * np.float32(0.001)).astype(np.float32)
    model = lib.default_model(n=n)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=burn, n_samples=keep, seed=seed)
    s = lib.create(model, hmc, lib.default_launch(), 1, 1)
    s.set_window_data(0, X, labels)
    s.init_chains(None)
    s.run(burn + keep)
    direct, tr = s.get_samples(0), s.get_traces(0)
    s.close()
    assert direct.tobytes() == data[0].tobytes()
    # and chain 0 against the oracle on those rows
    ref = orc.run_chain(ob.ref_model(n), ob.Hmc(L, burn, keep, burn, 0.01, 0.2, 0.1, 0.01, seed, 0), X, labels)
    lu = np.array([orc.log_uniform(seed, 0, t) for t in range(burn + keep)])
    clear = np.abs(lu - ref["log_acpt"]) > 1e-3
    assert np.array_equal(tr["accept"][clear], ref["accept"][clear])
    if clear.all():
        assert tr["eps"].tobytes() == ref["eps"].tobytes()
        np.testing.assert_allclose(direct, ref["samples"], rtol=0,
                                   atol=2e-4 * max(1.0, float(np.abs(ref["samples"]).max())))


# ------------------------------------------------------------------------------------------------
# a fixed group size makes a chain's bits independent of how the job is cut into calls
# ------------------------------------------------------------------------------------------------
def test_fixed_group_size_makes_call_boundaries_invisible(pkg, lib, orc):
    """More chains than fit at once (140 at 2 workgroups per chain; 128 fit), group size given: the chains
    run in fixed batches, every launch of a chain uses the same group size, so run(7) + run(6) equals run(13)
    bit for bit, and a chain saved after the first call and restored into a new sampler continues exactly.
    (With the automatic group size the left-over launches of a call run wider, and the bits then depend on
    where the calls end.)"""
    n, L, burn, keep, n_windows, seed = 512, 6, 4, 9, 140, 41
    model = lib.default_model(n=n, lik_scale=0.5, prior_scale=2.0)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=burn, n_samples=keep, eps0=0.01, seed=seed)
    launch = lib.default_launch(cus_per_chain=2, transitions_per_launch=5)

    def fresh():
        s = lib.create(model, hmc, launch, n_windows, 1)
        for w in range(n_windows):
            s.generate_window(w, teacher_scale=0.3, noise_sigma=0.5)
        s.init_chains(None)
        return s

    chains = (0, 1, 64, 127, 128, 139)
    a = fresh()
    a.run(13)
    whole = {c: (a.get_samples(c), a.get_chain_state(c), a.get_traces(c)) for c in chains}
    a.close()
    b = fresh()
    b.run(7)
    saved = {c: b.get_chain_state(c) for c in chains}
    b.run(6)
    for c in chains:
        st = b.get_chain_state(c)
        assert b.get_samples(c).tobytes() == whole[c][0].tobytes(), c
        assert st["w"].tobytes() == whole[c][1]["w"].tobytes() and st["grad"].tobytes() == whole[c][1]["grad"].tobytes()
        assert b.get_traces(c)["log_acpt"].tobytes() == whole[c][2]["log_acpt"].tobytes()
    b.close()
    # resume: a new sampler, the saved chains put back, the remaining six transitions
    r = fresh()
    for c in chains:
        st = saved[c]
        assert st["transitions_done"] == 7
        r.set_chain_state(c, st["w"], st["eps"], st["transitions_done"], st["n_accepted"])
    r.run(6)
    for c in chains:
        # (the other chains of r have run 6 transitions from their start: only the restored ones compare)
        got = r.get_samples(c)
        assert got[7 - burn:].tobytes() == whole[c][0][7 - burn:].tobytes(), c
        assert r.get_chain_state(c)["w"].tobytes() == whole[c][1]["w"].tobytes()
    r.close()


# ------------------------------------------------------------------------------------------------
# the exchange by slices: every wait is bounded, whichever rank stays away
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("G,drop", [(32, 3), (32, 31), (64, 5), (64, 62), (256, 200)])
def test_timeout_in_the_exchange_by_slices(pkg, lib, orc, monkeypatch, G, drop):
    """From 32 workgroups per chain on, the first workgroups of a group reduce one slice of the records each
    and everyone reads the totals.  A rank that never publishes (a reducing one: 3 of 31, 5 of 61; one that
    only contributes its record: 31, 62, 200) must end every other workgroup's wait at the spin limit: the
    call reports BNNHMC_ERR_TIMEOUT, every workgroup has exited, and the sampler works afterwards."""
    say("timeout G=%d withheld rank %d" % (G, drop))
    n = 16384
    model = lib.default_model(n=n)
    om = ob.ref_model(n)
    s = lib.create(model, lib.default_hmc(leapfrog_steps=5, burn_in=2, n_samples=2, seed=3),
                   lib.default_launch(cus_per_chain=G, spin_limit=2048), 1, 1)
    th = s.generate_window(0, teacher_scale=0.3, noise_sigma=5.0)
    X, y = s.get_window_data(0)
    monkeypatch.setenv("BNNHMC_DEBUG_DROP_ARRIVAL", str(drop))
    with pytest.raises(pkg.BnnHmcError) as e:
        s.eval(0, th)
    assert e.value.code == pkg.ERR_TIMEOUT and "spin limit" in str(e.value)
    with pytest.raises(pkg.BnnHmcError) as e:
        s.init_chains(None)
    assert e.value.code == pkg.ERR_TIMEOUT
    monkeypatch.delenv("BNNHMC_DEBUG_DROP_ARRIVAL")
    _, _, grad = s.eval(0, th)
    ref = orc.eval_f32(om, X, y, th)[2].astype(np.float64)
    assert float(np.abs(grad - ref).max()) <= 1e-5 * float(np.abs(ref).max())
    s.init_chains(None)
    s.run(4)
    assert s.get_chain_state(0)["transitions_done"] == 4
    s.close()


# ------------------------------------------------------------------------------------------------
# the step operator's failure record is sticky
# ------------------------------------------------------------------------------------------------
def test_step_operator_failure_record_survives_later_steps(pkg, lib, orc, monkeypatch):
    """Several steps queued on a stream, one check at the end: a step that failed must still be reported
    although steps that ran after it succeeded; the check clears the record, and the same workspace then
    serves further steps.  The workspace is handed over uninitialised (filled with a bit pattern)."""
    n, L, G = 4096, 3, 8
    model = lib.default_model(n=n)
    om = ob.ref_model(n)
    launch = lib.default_launch(cus_per_chain=G)
    X, y, th = orc.gen_window(1, 0, n, teacher_scale=0.3, noise_sigma=5.0)
    g0 = orc.eval_f32(om, X, y, th)[2]
    m0 = np.ones(P, np.float32)
    dev = DevBuf.from_numpy
    dX, dy, dw, dm, dg = dev(X), dev(y), dev(th), dev(m0), dev(g0)
    outs = [DevBuf.full(P, 0.0) for _ in range(4)]
    dloss = DevBuf.full(n + P, 0.0)
    wsb = lib.step_workspace_bytes(model, launch)
    ws = DevBuf.full(wsb // 4 + 16, 0x5A5A5A5A, np.uint32)   # as a fresh allocation might look

    def step():
        lib.mcmc_step(model, launch, dX.ptr, dy.ptr, dw.ptr, outs[0].ptr, dm.ptr, outs[1].ptr, dg.ptr,
                      outs[2].ptr, outs[3].ptr, dloss.ptr, ws.ptr, wsb, 0.01, L, 0)

    step()
    lib.step_check(model, launch, ws.ptr, 0)                 # garbage in the workspace is not an error
    monkeypatch.setenv("BNNHMC_DEBUG_PERTURB_HASH", "5")
    step()                                                   # this one reports a diverged workgroup ...
    monkeypatch.delenv("BNNHMC_DEBUG_PERTURB_HASH")
    step()                                                   # ... and two good ones follow
    step()
    with pytest.raises(pkg.BnnHmcError) as e:
        lib.step_check(model, launch, ws.ptr, 0)
    assert e.value.code == pkg.ERR_DIVERGED
    lib.step_check(model, launch, ws.ptr, 0)                 # reported once, then cleared
    step()
    lib.step_check(model, launch, ws.ptr, 0)
    ref = orc.mcmc_step(om, X, y, th, m0, g0, np.float32(0.01), L)
    assert float(np.abs(outs[2].numpy(P) - ref[2]).max()) <= 1e-5 * float(np.abs(ref[2]).max())


# ------------------------------------------------------------------------------------------------
# automatic batches: the rows of a launch within 1.4 times the memory-side cache, or as many chains as fit
# ------------------------------------------------------------------------------------------------
def test_automatic_batches_have_two_shapes_and_the_faster_is_measured(pkg, lib, orc, monkeypatch):
    """With the automatic group size a sampler starts with launches whose windows' rows stay within 358 MB:
    64 windows of 58368 x 22 (344 MB) on 4 workgroups each where 128 would fit the device on 2; chains that
    share a window share its rows (64 windows x 2 chains: 128 on 2); small windows are not cut.  A call long
    enough to hold a launch of each shape times both and goes on with the faster.  Whichever runs, only the
    layout over the device changes: the same transitions with the limit lifted (the measurement switch
    BNNHMC_RESIDENT_MB=0) or with the timing switched off (BNNHMC_BATCH_TUNE=0) take the same decisions and
    differ by the rounding of a different group size."""
    n_full = 58368
    # (a smooth posterior: with the benchmark's sigma = 0.01 log alpha is a difference of sums of order 1e8
    # and moves by 0.1 with the rounding of another group size)
    hmc = lib.default_hmc(leapfrog_steps=3, burn_in=0, n_samples=10, eps0=0.005, seed=9)
    model = lib.default_model(n=n_full, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=2.0, prior_scale=0.05)

    def run(n_windows, cpw, n_trans):
        s = lib.create(model, hmc, lib.default_launch(), n_windows, cpw)
        before = s.batching()
        for w in range(n_windows):
            s.generate_window(w, teacher_scale=0.1, noise_sigma=0.01)
        s.init_chains(None)
        s.run(n_trans)
        last = n_windows * cpw - 1
        out = dict(before=before, after=s.batching(), rates=s.batch_trial_rates(),
                   samples=[s.get_samples(c) for c in (0, last)], traces=[s.get_traces(c) for c in (0, last)])
        s.close()
        return out

    def same_chains(a, b, n_windows=128):
        for chain, x, y, tx, ty in zip((0, n_windows - 1), a["samples"], b["samples"], a["traces"], b["traces"]):
            # the same ratios and decisions, except where the uniform sits on the ratio (then neither the later
            # ratios nor the samples of that chain can be compared)
            close = [abs(orc.log_uniform(9, chain, k) - float(tx["log_acpt"][k])) < 0.02 for k in range(len(tx["accept"]))]
            if any(close):
                say("  chain %d: a uniform within 0.02 of the ratio, decisions not compared" % chain)
                continue
            assert np.allclose(tx["log_acpt"], ty["log_acpt"], rtol=2e-3, atol=1e-2), (tx["log_acpt"], ty["log_acpt"])
            assert np.array_equal(tx["accept"], ty["accept"])
            assert x.shape == y.shape and np.max(np.abs(x - y)) <= 1e-5 * np.max(np.abs(y))

    say("128 windows of 58368 rows, automatic group size, 10 transitions: both shapes are timed")
    tuned = run(128, 1, 10)              # 256 quanta of 5 transitions: one launch of 64, one of 128, then the faster
    assert tuned["before"] == (64, 4), tuned["before"]
    assert tuned["after"] in ((64, 4), (128, 2)), tuned["after"]
    assert tuned["rates"][0] > 0 and tuned["rates"][1] > 0
    say("  trial: %.0f evals/s within the row budget, %.0f evals/s device-wide -> %d x %d" % (
        tuned["rates"] + tuned["after"]))
    assert (tuned["after"] == (128, 2)) == (tuned["rates"][1] > tuned["rates"][0])
    short = run(128, 1, 2)               # no quantum of 5 transitions: nothing is timed
    assert short["after"] == (64, 4) and short["rates"] == (0.0, 0.0)
    monkeypatch.setenv("BNNHMC_BATCH_TUNE", "0")
    fixed = run(128, 1, 10)
    assert fixed["after"] == (64, 4) and fixed["rates"] == (0.0, 0.0)
    monkeypatch.delenv("BNNHMC_BATCH_TUNE")
    monkeypatch.setenv("BNNHMC_RESIDENT_MB", "0")
    wide = run(128, 1, 10)
    assert wide["before"] == wide["after"] == (128, 2) and wide["rates"] == (0.0, 0.0)
    monkeypatch.delenv("BNNHMC_RESIDENT_MB")
    same_chains(tuned, fixed)
    same_chains(wide, fixed)
    say("64 windows x 2 chains")
    s = lib.create(model, hmc, lib.default_launch(), 64, 2)
    assert s.batching() == (128, 2), s.batching()
    s.close()
    small = lib.default_model(n=4096, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=0.01, prior_scale=0.1)
    s = lib.create(small, hmc, lib.default_launch(), 200, 1)
    assert s.batching() == (128, 2), s.batching()
    s.close()
    s = lib.create(model, hmc, lib.default_launch(cus_per_chain=2), 200, 1)   # a configured group size is kept
    assert s.batching() == (128, 2), s.batching()
    s.close()
