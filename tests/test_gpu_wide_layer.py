"""GPU parity of the 64 -> 128 -> 1 network (P = 8449, the scaled benchmark shape): the LDS-resident
trajectory kernel, called through the C ABI, against the CPU oracle on the same seeded inputs.
Tolerances as for the 22 -> 40 -> 1 network: gradients and energies within 1e-5 relative, RNG
streams and decisions bit-exact."""
import sys

import numpy as np
import pytest

import orc_binding as ob
from hipmem import DevBuf

pytestmark = pytest.mark.gpu

D0, D1, P = 64, 128, 8449
RTOL = 1e-5


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def models(pkg, lib, kind, n):
    # teacher weights sized for O(1) pre-activations over 64 inputs (saturated tanh units cancel
    # catastrophically in any FP32 formulation of 1 - h^2)
    if kind == "t":
        return (lib.default_model(d0=D0, d1=D1, n=n), ob.Model(D0, D1, n, ob.LIK_STUDENT_T, 100.0, 2.2, 200.0),
                dict(teacher_scale=0.15, noise_sigma=5.0))
    if kind == "t_stiff":
        return (lib.default_model(d0=D0, d1=D1, n=n, lik_scale=0.5, prior_scale=2.0),
                ob.Model(D0, D1, n, ob.LIK_STUDENT_T, 0.5, 2.2, 2.0), dict(teacher_scale=0.15, noise_sigma=0.5))
    return (lib.default_model(d0=D0, d1=D1, n=n, lik_kind=pkg.LIK_GAUSSIAN, lik_scale=0.01, prior_scale=0.1),
            ob.Model(D0, D1, n, ob.LIK_GAUSSIAN, 0.01, 0.0, 0.1), dict(teacher_scale=0.05, noise_sigma=0.01))


def close_grad(a, b, what, rtol=RTOL):
    scale = float(np.abs(b).max())
    err = float(np.abs(a.astype(np.float64) - b).max())
    assert err <= rtol * scale + 1e-30, "%s: max abs err %.3e vs scale %.3e" % (what, err, scale)


def test_layer_sizes_are_checked(pkg, lib):
    assert lib.num_params(D0, D1) == P
    with pytest.raises(pkg.BnnHmcError):
        lib.create(lib.default_model(d0=64, d1=40, n=16), lib.default_hmc(), lib.default_launch(), 1, 1)
    with pytest.raises(pkg.BnnHmcError):  # no FFMA variant of the wide network
        lib.create(lib.default_model(d0=D0, d1=D1, n=16), lib.default_hmc(),
                   lib.default_launch(layer=pkg.LAYER_FFMA), 1, 1)
    with pytest.raises(pkg.BnnHmcError):  # at most 256 workgroups per chain
        lib.create(lib.default_model(d0=D0, d1=D1, n=16), lib.default_hmc(),
                   lib.default_launch(cus_per_chain=512), 1, 1)


@pytest.mark.parametrize("kind", ["t", "gauss"])
@pytest.mark.parametrize("n,G", [(1, 1), (3, 2), (16, 1), (17, 4), (100, 3), (1000, 8), (4101, 32),
                                 (9000, 64), (58368, 0), (233472, 64), (9000, 96), (40000, 128), (233472, 256)])
def test_eval_matches_oracle(pkg, lib, orc, kind, n, G):
    say("wide eval lik=%s n=%d G=%d" % (kind, n, G))
    model, om, gen = models(pkg, lib, kind, n)
    s = lib.create(model, lib.default_hmc(seed=n), lib.default_launch(cus_per_chain=G), 1, 1)
    th = s.generate_window(0, **gen)
    X, y = s.get_window_data(0)
    Xo, yo, tho = orc.gen_window(n, 0, n, d0=D0, d1=D1, **gen)
    assert X.tobytes() == Xo.tobytes() and y.tobytes() == yo.tobytes() and th.tobytes() == tho.tobytes()
    rng = np.random.default_rng(n)
    for w in (np.zeros(P, np.float32), (th * 0.7 + rng.normal(0, 0.02 * gen["teacher_scale"], P)).astype(np.float32)):
        ell, prior, grad = s.eval(0, w)
        ell_o, prior_o, grad_o, _ = orc.eval_f32(om, X, y, w)
        _, _, grad64 = orc.eval_f64(om, X, y, w.astype(np.float64))
        close_grad(grad, grad_o, "grad vs f32 oracle")
        close_grad(grad, grad64, "grad vs f64 oracle", rtol=2e-5)
        np.testing.assert_allclose(ell, ell_o, rtol=RTOL, atol=RTOL * max(1.0, float(np.abs(ell_o).max())))
        assert prior.tobytes() == prior_o.tobytes()
        U, Uo = -(ell.sum(dtype=np.float64) + prior.sum(dtype=np.float64)), -(
            ell_o.sum(dtype=np.float64) + prior_o.sum(dtype=np.float64))
        assert abs(U - Uo) <= RTOL * abs(Uo)
    s.close()


def test_eval_is_deterministic(pkg, lib, orc):
    n = 5000
    model, om, gen = models(pkg, lib, "t", n)
    outs = {}
    for G in (1, 4, 32):
        for rep in range(2):
            s = lib.create(model, lib.default_hmc(seed=3), lib.default_launch(cus_per_chain=G), 1, 1)
            th = s.generate_window(0, **gen)
            _, _, grad = s.eval(0, th)
            s.close()
            if rep == 0:
                outs[G] = grad
            else:
                assert grad.tobytes() == outs[G].tobytes(), "two runs differ at G=%d" % G
    close_grad(outs[1], outs[32].astype(np.float64), "G=1 vs G=32", rtol=3e-6)
    close_grad(outs[4], outs[32].astype(np.float64), "G=4 vs G=32", rtol=3e-6)


@pytest.mark.parametrize("kind,n,L,eps,G,offset", [("t", 777, 1, 0.01, 4, 0), ("t", 2048, 2, 0.01, 8, 0),
                                                   ("t", 1500, 25, 0.003, 32, 0), ("gauss", 999, 10, 1e-5, 5, 0),
                                                   ("gauss", 4096, 40, 1e-5, 64, 0), ("t", 20000, 12, 0.003, 0, 0),
                                                   ("t", 333, 3, 0.01, 2, 4), ("t", 30000, 10, 0.003, 128, 0),
                                                   ("gauss", 58368, 6, 1e-5, 256, 0)])
def test_mcmc_step_operator_matches_oracle(pkg, lib, orc, kind, n, L, eps, G, offset):
    say("wide mcmc_step lik=%s n=%d L=%d G=%d offset=%d" % (kind, n, L, G, offset))
    model, om, gen = models(pkg, lib, kind, n)
    launch = lib.default_launch(cus_per_chain=G)
    X, y, th = orc.gen_window(5, 1, n, d0=D0, d1=D1, **gen)
    rng = np.random.default_rng(n + L)
    w0 = (th * 0.8).astype(np.float32)
    m0 = rng.normal(0, 1, P).astype(np.float32)
    g0 = orc.eval_f32(om, X, y, w0)[2]
    dev = DevBuf.from_numpy
    dX, dy = dev(X, offset_bytes=offset), dev(y, offset_bytes=3 * offset)  # offset: unaligned caller buffers
    dw0, dm0, dg0 = dev(w0), dev(m0), dev(g0)
    dw1, dm1, dg1, dgn = (DevBuf.full(P, np.nan) for _ in range(4))
    dloss = DevBuf.full(n + P, np.nan)
    wsb = lib.step_workspace_bytes(model, launch)
    ws = DevBuf.full(wsb // 4 + 16, 0, np.int32)
    st = 0
    lib.mcmc_step(model, launch, dX.data_ptr, dy.data_ptr, dw0.ptr, dw1.ptr, dm0.ptr, dm1.ptr, dg0.ptr,
                  dg1.ptr, dgn.ptr, dloss.ptr, ws.ptr, wsb, eps, L, st)
    lib.step_check(model, launch, ws.ptr, st)
    w1, m1, g1 = dw1.numpy(P), dm1.numpy(P), dg1.numpy(P)
    loss = dloss.numpy(n + P)
    w1o, m1o, g1o, losso = orc.mcmc_step(om, X, y, w0, m0, g0, eps, L)
    assert np.all(dgn.numpy(P) == 0)
    np.testing.assert_allclose(w1, w1o, rtol=0, atol=1e-6 * L * max(1.0, float(np.abs(w1o).max())))
    np.testing.assert_allclose(m1, m1o, rtol=0, atol=3e-6 * L * max(1.0, float(np.abs(m1o).max())))
    close_grad(g1, g1o.astype(np.float64), "grad_cur", rtol=RTOL * max(1, L // 4))
    np.testing.assert_allclose(loss[:n], losso[:n], rtol=1e-5 * max(1, L // 4),
                               atol=1e-5 * max(1, L // 4) * max(1.0, float(np.abs(losso[:n]).max())))
    np.testing.assert_allclose(loss[n:], losso[n:], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("G", [8, 128])
def test_transitions_match_oracle_decisions(pkg, lib, orc, G):
    """G = 8: every workgroup adds all records; G = 128: the two-phase exchange (each workgroup reduces
    slices of the parameters, all read the totals)."""
    n, L, burn, keep, seed = 1024, 12, 20, 20, 33
    model, om, gen = models(pkg, lib, "t_stiff", n)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=burn, n_samples=keep, eps0=0.004, seed=seed)
    s = lib.create(model, hmc, lib.default_launch(cus_per_chain=G, transitions_per_launch=7), 1, 1)
    s.generate_window(0, **gen)
    X, y = s.get_window_data(0)
    s.init_chains(None)
    s.run(burn + keep)
    tr, state, samples = s.get_traces(0), s.get_chain_state(0), s.get_samples(0)
    l1, l2, fl = s.final_loss(0)
    s.close()
    ref = orc.run_chain(om, ob.Hmc(L, burn, keep, burn, 0.004, 0.2, 0.1, 0.01, seed, 0), X, y)
    T = burn + keep
    say("wide transitions: %d/%d accepted (oracle %d)" % (tr["accept"].sum(), T, ref["accept"].sum()))
    margin = np.abs(np.array([orc.log_uniform(seed, 0, t) for t in range(T)]) - ref["log_acpt"])
    assert margin.min() > 1e-3, "test inputs put a decision on a knife edge"
    assert np.array_equal(tr["accept"], ref["accept"])
    assert 0 < ref["accept"].sum() < T
    np.testing.assert_allclose(tr["log_acpt"], ref["log_acpt"], rtol=2e-3, atol=5e-3)
    assert tr["eps"].tobytes() == ref["eps"].tobytes()
    assert state["n_accepted"] == ref["n_accept"] and state["transitions_done"] == T
    np.testing.assert_allclose(samples, ref["samples"], rtol=0,
                               atol=2e-4 * max(1.0, float(np.abs(ref["samples"]).max())))
    for t in range(burn + 1, T):
        if not tr["accept"][t]:
            assert np.array_equal(samples[t - burn], samples[t - burn - 1])
    o1, o2, ofl = orc.final_loss(om, X, y, samples)
    assert l1 == pytest.approx(o1, rel=1e-5) and l2 == pytest.approx(o2, rel=1e-6)
    assert fl == pytest.approx(ofl, rel=1e-5)


def test_windows_times_four_chains_are_independent_and_reproducible(pkg, lib, orc):
    # the scaled shape runs 4 chains per window: chains of a window share its rows and differ in
    # their RNG streams; a chain's output does not depend on what else is in the batch
    n, L, T = 600, 6, 6
    model, om, gen = models(pkg, lib, "t_stiff", n)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=2, n_samples=T - 2, eps0=0.004, seed=9)

    def run(windows, cpw, G):
        s = lib.create(model, hmc, lib.default_launch(cus_per_chain=G), windows, cpw)
        for w in range(windows):
            s.generate_window(w, **gen)
        s.init_chains(None)
        s.run(T)
        out = [s.get_samples(c) for c in range(windows * cpw)]
        s.close()
        return out

    a = run(3, 4, 4)
    b = run(3, 4, 4)
    for c in range(12):
        assert a[c].tobytes() == b[c].tobytes()
    assert not np.array_equal(a[0], a[1])      # same window, different chain
    assert not np.array_equal(a[0], a[4])      # different window
    # chain 0 of window 0 against the oracle's chain with the same identifiers
    X, y, _ = orc.gen_window(9, 0, n, d0=D0, d1=D1, **gen)
    ref = orc.run_chain(om, ob.Hmc(L, 2, T - 2, 2, 0.004, 0.2, 0.1, 0.01, 9, 0), X, y)
    np.testing.assert_allclose(a[0], ref["samples"], rtol=0,
                               atol=2e-4 * max(1.0, float(np.abs(ref["samples"]).max())))


def test_window_diagnostics_use_the_four_chains(pkg, lib, orc):
    n, L, burn, keep = 400, 5, 2, 10
    model, om, gen = models(pkg, lib, "t_stiff", n)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=burn, n_samples=keep, eps0=0.004, seed=4)
    s = lib.create(model, hmc, lib.default_launch(cus_per_chain=4), 2, 4)
    for w in range(2):
        s.generate_window(w, **gen)
    s.init_chains(None)
    s.run(burn + 4)
    with pytest.raises(pkg.BnnHmcError):       # four kept samples so far: too few
        s.diagnostics(1)
    s.run(keep - 4)
    rhat, ess = s.diagnostics(1)
    chains = np.stack([s.get_samples(4 + c) for c in range(4)])
    s.close()
    r_host, e_host = lib.split_rhat_ess(chains)
    assert rhat.tobytes() == r_host.tobytes() and ess.tobytes() == e_host.tobytes()
    assert np.all(np.isfinite(rhat)) and np.all(rhat >= 0.5) and np.all(ess > 0)


def test_one_transition_at_full_size(pkg, lib, orc):
    """The scaled shape at its stated size (64 -> 128 -> 1, 233472 rows, 4 workgroups per chain as the
    batched job runs it): one whole transition of 50 leapfrog steps from the all-zero start with the
    reference's model constants and eps0 = 0.01, against the oracle: log accept ratio, decision, the state
    the chain ends in and the step size after adaptation."""
    n, L = 233472, 50
    say("64->128->1, one transition of %d leapfrog steps on %d rows" % (L, n))
    model = lib.default_model(d0=D0, d1=D1, n=n)
    om = ob.Model(D0, D1, n, ob.LIK_STUDENT_T, 100.0, 2.2, 200.0)
    hmc = lib.default_hmc(leapfrog_steps=L, burn_in=1, n_samples=1, eps0=0.01, seed=6)
    s = lib.create(model, hmc, lib.default_launch(cus_per_chain=4), 1, 1)
    s.generate_window(0, teacher_scale=0.05, noise_sigma=0.01)
    X, y = s.get_window_data(0)
    s.init_chains(None)
    s.run(1)
    tr, st = s.get_traces(0), s.get_chain_state(0)
    s.close()
    ref = orc.run_chain_from(om, ob.Hmc(L, 1, 1, 1, 0.01, 0.2, 0.1, 0.01, 6, 0), X, y, None, 0.01, 0, 1)
    lu = orc.log_uniform(6, 0, 0)
    say("log accept ratio: gpu %.6g oracle %.6g, log u %.4f, accepted %d %d" % (
        tr["log_acpt"][0], ref["log_acpt"][0], lu, tr["accept"][0], ref["accept"][0]))
    # a sum of 233472 differences of per-row terms of size 5.6, each known to one FP32 ulp (4.8e-7):
    # 2.3e-4 of rounding noise at random signs in either implementation
    assert abs(float(tr["log_acpt"][0]) - float(ref["log_acpt"][0])) <= 6e-4
    assert abs(lu - float(ref["log_acpt"][0])) > 1e-2, "the inputs put the decision on a knife edge"
    assert tr["accept"][0] == ref["accept"][0] == 1
    assert np.float32(tr["eps"][0]).tobytes() == np.float32(ref["eps"][0]).tobytes()
    np.testing.assert_allclose(st["w"], ref["final_w"], rtol=0,
                               atol=1e-6 * L * max(1.0, float(np.abs(ref["final_w"]).max())))
    assert float(np.abs(ref["final_w"]).max()) > 0.5         # the chain did move
