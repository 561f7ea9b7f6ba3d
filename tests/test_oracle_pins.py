"""Pins the CPU oracle against evidence that is independent of it.

The reference ships no tests or golden vectors, so each oracle function is pinned by published
known-answer vectors (Philox), library routines (scipy / numpy / torch.autograd), closed forms and
invariants, chosen so that a dropped term, a wrong sign or index, or a transposed operand fails.
"""
import math

import numpy as np
import pytest
import scipy.special
import scipy.stats

import orc_binding as ob

D0, D1 = 22, 40
P = D0 * D1 + 2 * D1 + 1


# ----------------------------------------------------------------------------------------------
# constants (global_params.h:39-52)
# ----------------------------------------------------------------------------------------------
def test_layout_and_param_count(orc):
    assert orc.num_params(22, 40) == 961  # global_params.h:57-58
    assert orc.num_params(64, 128) == 8449


def test_reference_normalisation_constants(orc):
    m = ob.ref_model(n=1)
    # y == yhat + b2  =>  log-lik = -STUDENT_T_LOSS_NORMALIZATION (global_params.h:45)
    ell, g = orc.row_loglik(m, 0.25, 0.2, 0.05)
    assert abs(0.25 - 0.2 - 0.05) < 1e-7
    assert np.float32(ell) == pytest.approx(-5.63448313353184, abs=6e-7)
    lp, gp = orc.prior_terms(m, 0.0)
    assert np.float32(lp) == np.float32(-6.21725589975271)  # global_params.h:52
    assert gp == 0.0
    # the closed forms quoted in global_params.h:41-44 and :51
    closed = (math.log(100.0) + 0.5 * math.log(2.2) + 0.5 * math.log(math.pi) + math.lgamma(1.1)
              - math.lgamma(1.6))
    assert closed == pytest.approx(5.63448313353184, abs=1e-13)
    assert np.float32(closed) == np.float32(5.63448313353184)
    assert 0.5 * math.log(2 * math.pi) + math.log(200.0) == pytest.approx(6.21725589975271, abs=1e-13)
    # prior gradient uses -1/scale^2 = -0.000025 (global_params.h:50)
    _, gp = orc.prior_terms(m, 3.0)
    assert np.float32(gp) == np.float32(3.0) * np.float32(-0.000025)


# ----------------------------------------------------------------------------------------------
# RNG
# ----------------------------------------------------------------------------------------------
def test_philox_known_answers(orc):
    # Random123 kat_vectors, philox4x32 with 10 rounds
    assert orc.philox([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert orc.philox([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6,
                                                             0x6D5451FD]
    assert orc.philox([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344],
                      [0xA4093822, 0x299F31D0]) == [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_rng_word_counter_mapping(orc):
    # word `index` is word index%4 of the block with counter (index/4, t, stream, 0), key (seed, id)
    for idx in (0, 1, 5, 962, 1284095):
        blk = orc.philox([idx // 4, 7, ob.STREAM_MOMENTUM, 0], [11, 3])
        assert orc.rng_word(11, 3, ob.STREAM_MOMENTUM, 7, idx) == blk[idx % 4]
    # different streams / transitions / chains give different words
    base = orc.rng_word(0, 0, 3, 0, 0)
    assert len({base, orc.rng_word(0, 0, 4, 0, 0), orc.rng_word(0, 0, 3, 1, 0),
                orc.rng_word(0, 1, 3, 0, 0), orc.rng_word(1, 0, 3, 0, 0)}) == 5


def test_det_log_and_sqrt_match_libm(orc):
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.uniform(2.0 ** -33, 1.0, 2000), 2.0 ** rng.uniform(-40, 40, 2000),
                         [2.0 ** -33, 0.5, 1.0 - 2.0 ** -53, 1.0, 1.5, math.sqrt(2) / 2, math.sqrt(2)]])
    for x in xs:
        ref = math.log(x)
        assert abs(orc.det_log(x) - ref) <= 2.3e-16 * max(abs(ref), 1e-300) + 1e-17 * 0
        s = orc.det_sqrt(x)
        assert abs(s - math.sqrt(x)) <= 2.3e-16 * math.sqrt(x)


def test_ppnd16_matches_scipy_ndtri(orc):
    ps = np.concatenate([np.linspace(1e-9, 1 - 1e-9, 4001), 10.0 ** -np.arange(1, 11.0),
                         1 - 10.0 ** -np.arange(1, 11.0), [0.5, 0.075, 0.925, 0.0751, 0.9249,
                                                           (0.5) * 2.0 ** -32]])
    for p in ps:
        ref = scipy.special.ndtri(p)
        assert abs(orc.ppnd16(p) - ref) <= 1e-13 * max(1.0, abs(ref)), p
    assert orc.ppnd16(0.5) == 0.0
    assert orc.ppnd16(0.3) == -orc.ppnd16(0.7) or abs(orc.ppnd16(0.3) + orc.ppnd16(0.7)) < 1e-15


def test_normal_stream_statistics(orc):
    n = 200_000
    z = np.array([orc.normal(5, 2, ob.STREAM_MOMENTUM, 9, i) for i in range(n)], np.float64)
    assert abs(z.mean()) < 4 / math.sqrt(n)
    assert abs(z.var() - 1) < 4 * math.sqrt(2 / n)
    assert abs(scipy.stats.skew(z)) < 4 * math.sqrt(6 / n)
    assert abs(scipy.stats.kurtosis(z)) < 4 * math.sqrt(24 / n)
    assert scipy.stats.kstest(z, "norm").pvalue > 1e-3
    # momentum() is exactly this stream
    mom = orc.momentum(5, 2, 9, 961)
    assert np.array_equal(mom, z[:961].astype(np.float32))
    # the value is the quantile of (word + 0.5) / 2^32
    k = orc.rng_word(5, 2, ob.STREAM_MOMENTUM, 9, 17)
    assert np.float32(scipy.special.ndtri((k + 0.5) / 2 ** 32)) == pytest.approx(mom[17], rel=3e-7)


def test_log_uniform(orc):
    vals = []
    for t in range(2000):
        k = orc.rng_word(3, 1, ob.STREAM_ACCEPT, t, 0)
        lu = orc.log_uniform(3, 1, t)
        assert lu == np.float32(math.log((k + 0.5) / 2 ** 32)) or abs(
            lu - math.log((k + 0.5) / 2 ** 32)) < 2e-7 * abs(lu) + 1e-9
        assert lu < 0
        vals.append(math.exp(lu))
    assert scipy.stats.kstest(vals, "uniform").pvalue > 1e-3


# ----------------------------------------------------------------------------------------------
# scalar pieces
# ----------------------------------------------------------------------------------------------
def test_tanh_forward_backward(orc):
    xs = np.concatenate([np.linspace(-12, 12, 4001), np.linspace(-0.01, 0.01, 401),
                         [0.0048176, 0.0048177, -0.0048176, -0.0048177, 40.0, -40.0, 100.0, -100.0]])
    for x in xs.astype(np.float32):
        out = orc.tanh_fwd(float(x))
        ref = math.tanh(float(x))
        if abs(x) < 0.0048176045529544353485:
            assert out == x  # identity branch, kernel_helpers.h:41
            assert abs(out - ref) <= abs(float(x)) ** 3 / 3 + 1e-12
        else:
            # cancellation in 2*sigmoid - 1 leaves an absolute error of a few float ulps of 1
            assert abs(out - ref) <= 2.5e-7
    # backward is (1 - out^2) * dgrad (kernel_helpers.h:43)
    for out, dg in [(0.0, 1.0), (0.5, 2.0), (-0.9, -3.0), (1.0, 5.0)]:
        assert orc.tanh_bwd(out, dg) == pytest.approx((1 - out * out) * dg, rel=2e-7, abs=1e-12)


@pytest.mark.parametrize("scale,df", [(100.0, 2.2), (1.0, 5.0), (0.3, 1.0)])
def test_student_t_row_loglik(orc, scale, df):
    m = ob.Model(D0, D1, 1, ob.LIK_STUDENT_T, scale, df, 200.0)
    rng = np.random.default_rng(1)
    for _ in range(200):
        y, yhat, b2 = rng.normal(0, 3 * scale, 3)
        ell, g = orc.row_loglik(m, y, yhat, b2)
        loc = float(np.float32(yhat)) + float(np.float32(b2))
        yf = float(np.float32(y))
        ref = scipy.stats.t.logpdf(yf, df, loc=loc, scale=scale)
        assert ell == pytest.approx(ref, rel=3e-6, abs=3e-6)
        h = 1e-4 * scale
        fd = (scipy.stats.t.logpdf(yf, df, loc=loc + h, scale=scale)
              - scipy.stats.t.logpdf(yf, df, loc=loc - h, scale=scale)) / (2 * h)
        assert g == pytest.approx(fd, rel=2e-5, abs=2e-6 / scale)


def test_gaussian_row_loglik(orc):
    m = ob.gauss_model(n=1, sigma=0.01)
    rng = np.random.default_rng(2)
    for _ in range(200):
        y, yhat, b2 = rng.normal(0, 0.05, 3)
        ell, g = orc.row_loglik(m, y, yhat, b2)
        loc = float(np.float32(yhat)) + float(np.float32(b2))
        yf = float(np.float32(y))
        ref = scipy.stats.norm.logpdf(yf, loc=loc, scale=0.01)
        assert ell == pytest.approx(ref, rel=2e-5, abs=2e-5)
        assert g == pytest.approx((yf - loc) / 1e-4, rel=2e-5, abs=1e-3)


def test_prior_terms(orc):
    for scale in (200.0, 0.1):
        m = ob.Model(D0, D1, 1, ob.LIK_STUDENT_T, 100.0, 2.2, scale)
        for w in (-3.0, -0.01, 0.0, 0.2, 7.5):
            lp, gp = orc.prior_terms(m, w)
            assert lp == pytest.approx(scipy.stats.norm.logpdf(w, scale=scale), rel=2e-6, abs=2e-6)
            assert gp == pytest.approx(-w / scale ** 2, rel=2e-6, abs=1e-12)


# ----------------------------------------------------------------------------------------------
# log-posterior and gradient
# ----------------------------------------------------------------------------------------------
def _numpy_forward(X, w, d0=D0, d1=D1):
    W1 = w[:d0 * d1].reshape(d0, d1)          # index k*D1 + c (ffma.h:35-44)
    b1 = w[d0 * d1:d0 * d1 + d1]
    w2 = w[d0 * d1 + d1:d0 * d1 + 2 * d1]
    b2 = w[-1]
    H = np.tanh(X.astype(np.float64) @ W1 + b1)
    return H @ w2, b2, H


def _torch_logpost_grad(m, X, y, w):
    import torch

    d0, d1 = m.d0, m.d1

    def f64(v):
        return torch.tensor(v, dtype=torch.float64)

    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    Xt = torch.tensor(X, dtype=torch.float64)
    yt = torch.tensor(y, dtype=torch.float64)
    W1 = wt[:d0 * d1].reshape(d0, d1)
    b1 = wt[d0 * d1:d0 * d1 + d1]
    w2 = wt[d0 * d1 + d1:d0 * d1 + 2 * d1]
    b2 = wt[-1]
    mu = torch.tanh(Xt @ W1 + b1) @ w2 + b2
    if m.lik_kind == ob.LIK_STUDENT_T:
        lik = torch.distributions.StudentT(f64(m.lik_df), mu, f64(m.lik_scale)).log_prob(yt)
    else:
        lik = torch.distributions.Normal(mu, f64(m.lik_scale)).log_prob(yt)
    prior = torch.distributions.Normal(f64(0.0), f64(m.prior_scale)).log_prob(wt)
    total = lik.sum() + prior.sum()
    total.backward()
    return lik.detach().numpy(), prior.detach().numpy(), wt.grad.numpy()


def _case(orc, n, lik, seed):
    X, y, th = orc.gen_window(seed, 0, n)
    rng = np.random.default_rng(seed)
    if lik == "t":
        m = ob.Model(D0, D1, n, ob.LIK_STUDENT_T, 0.5, 2.2, 2.0)
    else:
        m = ob.gauss_model(n=n, sigma=0.05, prior=0.3)
    w = (th + rng.normal(0, 0.05, P)).astype(np.float32)
    return m, X, y, w


@pytest.mark.parametrize("lik", ["t", "gauss"])
@pytest.mark.parametrize("n", [1, 3, 17, 64, 1000])
def test_eval_against_torch_autograd(orc, lik, n):
    m, X, y, w = _case(orc, n, lik, seed=10 + n)
    lik_t, prior_t, grad_t = _torch_logpost_grad(m, X, y, w.astype(np.float64))
    ell64, prior64, grad64 = orc.eval_f64(m, X, y, w.astype(np.float64))
    np.testing.assert_allclose(ell64, lik_t, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(prior64, prior_t, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(grad64, grad_t, rtol=1e-9, atol=1e-9 * np.abs(grad_t).max())
    ell32, prior32, grad32, yhat32 = orc.eval_f32(m, X, y, w)
    yh_np, _, _ = _numpy_forward(X, w.astype(np.float64))
    np.testing.assert_allclose(yhat32, yh_np, rtol=0, atol=2e-6)
    gmax = np.abs(grad_t).max()
    np.testing.assert_allclose(grad32, grad_t, rtol=2e-5, atol=2e-5 * gmax)
    np.testing.assert_allclose(ell32, lik_t, rtol=2e-5, atol=2e-5 * max(1.0, np.abs(lik_t).max()))
    np.testing.assert_allclose(prior32, prior_t, rtol=1e-6, atol=1e-6)


def test_eval_gradient_finite_differences(orc):
    # all 961 parameters, central differences of the float64 log-posterior, tiny N
    m, X, y, w = _case(orc, 8, "t", seed=3)
    w64 = w.astype(np.float64)
    _, _, grad = orc.eval_f64(m, X, y, w64)
    h = 1e-6
    for p in range(P):
        wp, wm = w64.copy(), w64.copy()
        wp[p] += h
        wm[p] -= h
        ep, pp, _ = orc.eval_f64(m, X, y, wp)
        em, pm, _ = orc.eval_f64(m, X, y, wm)
        fd = ((ep.sum() + pp.sum()) - (em.sum() + pm.sum())) / (2 * h)
        assert grad[p] == pytest.approx(fd, rel=2e-6, abs=2e-7), p


def test_eval_at_zero_weights_is_closed_form(orc):
    # the reference's actual initial state (main.h:52, 182): h = 0, yhat = 0
    n = 500
    m = ob.ref_model(n=n)
    X, y, _ = orc.gen_window(4, 0, n, teacher_scale=30.0, noise_sigma=5.0)
    w = np.zeros(P, np.float32)
    ell, prior, grad, yhat = orc.eval_f32(m, X, y, w)
    assert np.all(yhat == 0)
    assert np.all(grad[:P - 1] == 0)  # W1, b1, w2 gradients vanish exactly
    d = y.astype(np.float64) / 100.0
    np.testing.assert_allclose(ell, scipy.stats.t.logpdf(y.astype(np.float64), 2.2, scale=100.0),
                               rtol=2e-6)
    assert grad[-1] == pytest.approx(np.sum(d * 3.2 / 100.0 / (d * d + 2.2)), rel=1e-6)
    assert prior.sum(dtype=np.float64) == pytest.approx(-961 * 6.21725589975271, rel=1e-7)


def test_eval_is_a_sum_over_rows(orc):
    # permuting rows changes the gradient only by rounding; splitting rows adds likelihood parts
    m, X, y, w = _case(orc, 256, "gauss", seed=7)
    _, _, g_all, _ = orc.eval_f32(m, X, y, w)
    perm = np.random.default_rng(0).permutation(256)
    _, _, g_perm, _ = orc.eval_f32(m, X[perm], y[perm], w)
    np.testing.assert_allclose(g_perm, g_all, rtol=0, atol=3e-6 * np.abs(g_all).max())
    ma = ob.gauss_model(n=100, sigma=0.05, prior=0.3)
    mb = ob.gauss_model(n=156, sigma=0.05, prior=0.3)
    _, _, ga, _ = orc.eval_f32(ma, X[:100], y[:100], w)
    _, _, gb, _ = orc.eval_f32(mb, X[100:], y[100:], w)
    prior_g = np.array([orc.prior_terms(m, float(v))[1] for v in w], np.float64)
    np.testing.assert_allclose(ga.astype(np.float64) + gb - prior_g, g_all, rtol=0,
                               atol=3e-6 * np.abs(g_all).max())


def test_eval_layout_is_k_major(orc):
    # W1 index is k*D1 + c: perturbing W1[k=2][c=5] must change only hidden unit 5's pre-activation
    n = 4
    m = ob.gauss_model(n=n)
    X = np.zeros((n, D0), np.float32)
    X[:, 2] = 1.0
    y = np.zeros(n, np.float32)
    w = np.zeros(P, np.float32)
    w[2 * D1 + 5] = 0.7             # W1[2][5]
    w[D0 * D1 + D1 + 5] = 1.0       # w2[5]
    _, _, _, yhat = orc.eval_f32(m, X, y, w)
    np.testing.assert_allclose(yhat, math.tanh(0.7), rtol=1e-6)
    w[D0 * D1 + D1 + 5] = 0.0
    w[D0 * D1 + D1 + 6] = 1.0       # w2[6] sees nothing
    _, _, _, yhat = orc.eval_f32(m, X, y, w)
    assert np.all(yhat == 0)


# ----------------------------------------------------------------------------------------------
# leapfrog (ffma.h:106-120, 395-427)
# ----------------------------------------------------------------------------------------------
def test_leapfrog_prior_only_is_harmonic_oscillator(orc):
    # no rows: log pi = -w^2 / (2 s^2), the exact flow is a rotation with omega = 1/s
    s = 2.0
    m = ob.Model(D0, D1, 0, ob.LIK_STUDENT_T, 100.0, 2.2, s)
    rng = np.random.default_rng(5)
    w0 = rng.normal(0, 1, P).astype(np.float32)
    m0 = rng.normal(0, 1, P).astype(np.float32)
    g0 = (-w0.astype(np.float64) / s ** 2).astype(np.float32)
    X = np.zeros((0, D0), np.float32)
    y = np.zeros(0, np.float32)
    eps, L = 0.01, 300
    w1, m1, g1, loss = orc.mcmc_step(m, X, y, w0, m0, g0, eps, L)
    # m1 lacks the final half kick (kernel_helpers.h:169-171)
    m_full = m1.astype(np.float64) + 0.5 * eps * g1
    t = eps * L
    om = 1 / s
    w_exact = w0 * math.cos(om * t) + m0 * s * math.sin(om * t)
    m_exact = m0 * math.cos(om * t) - w0 / s * math.sin(om * t)
    # leapfrog global error is O(eps^2 t omega^3); 3e-5 here
    np.testing.assert_allclose(w1, w_exact, atol=2e-4)
    np.testing.assert_allclose(m_full, m_exact, atol=2e-4)
    np.testing.assert_allclose(g1, -w1.astype(np.float64) / s ** 2, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(loss, scipy.stats.norm.logpdf(w1.astype(np.float64), scale=s), rtol=2e-6)


def _textbook_leapfrog(orc, m, X, y, w, mom, eps, L):
    """half kick, (drift, full kick) x (L-1), drift, half kick -- in float64 on the oracle gradient"""
    w = w.astype(np.float64).copy()
    mom = mom.astype(np.float64).copy()
    g = orc.eval_f64(m, X, y, w)[2]
    mom += 0.5 * eps * g
    for s in range(L):
        w += eps * mom
        g = orc.eval_f64(m, X, y, w)[2]
        mom += (eps if s < L - 1 else 0.5 * eps) * g
    return w, mom, g


def test_mcmc_step_equals_textbook_leapfrog(orc):
    m, X, y, w = _case(orc, 64, "t", seed=8)
    rng = np.random.default_rng(8)
    mom = rng.normal(0, 1, P).astype(np.float32)
    g0 = orc.eval_f32(m, X, y, w)[2]
    eps, L = 2e-3, 25
    w1, m1, g1, loss = orc.mcmc_step(m, X, y, w, mom, g0, eps, L)
    wt, mt, gt = _textbook_leapfrog(orc, m, X, y, w, mom, eps, L)
    np.testing.assert_allclose(w1, wt, atol=5e-6)
    np.testing.assert_allclose(m1.astype(np.float64) + 0.5 * eps * g1, mt, atol=2e-4)
    np.testing.assert_allclose(g1, gt, rtol=1e-4, atol=1e-4 * np.abs(gt).max())
    ell, prior, _, _ = orc.eval_f32(m, X, y, w1)
    np.testing.assert_array_equal(loss[:64], ell)      # only the last step records them
    np.testing.assert_array_equal(loss[64:], prior)
    # L = 1 with eps = 0 is a pure evaluation (main.h:96-99)
    w2, m2, g2, loss2 = orc.mcmc_step(m, X, y, w, np.zeros(P), np.zeros(P), 0.0, 1)
    np.testing.assert_array_equal(w2, w)
    np.testing.assert_array_equal(g2, g0)


def test_mcmc_step_is_time_reversible(orc):
    m, X, y, w = _case(orc, 64, "gauss", seed=9)
    mom = np.random.default_rng(9).normal(0, 1, P).astype(np.float32)
    g0 = orc.eval_f32(m, X, y, w)[2]
    eps, L = 2e-4, 40
    w1, m1, g1, _ = orc.mcmc_step(m, X, y, w, mom, g0, eps, L)
    m1_full = (m1 + np.float32(0.5 * eps) * g1).astype(np.float32)
    w2, m2, g2, _ = orc.mcmc_step(m, X, y, w1, -m1_full, g1, eps, L)
    m2_full = m2 + np.float32(0.5 * eps) * g2
    np.testing.assert_allclose(w2, w, atol=3e-5)
    np.testing.assert_allclose(-m2_full, mom, atol=2e-3)


def _hamiltonian64(orc, m, X, y, w, mom_full):
    ell, prior, _ = orc.eval_f64(m, X, y, np.asarray(w, np.float64))
    return -(ell.sum() + prior.sum()) + 0.5 * np.sum(np.asarray(mom_full, np.float64) ** 2)


def test_energy_error_is_second_order(orc):
    m, X, y, w = _case(orc, 128, "t", seed=11)
    mom = np.random.default_rng(11).normal(0, 1, P).astype(np.float32)
    g0 = orc.eval_f32(m, X, y, w)[2]
    H0 = _hamiltonian64(orc, m, X, y, w, mom)
    errs = []
    for eps, L in [(8e-3, 25), (4e-3, 50), (2e-3, 100)]:
        w1, m1, g1, _ = orc.mcmc_step(m, X, y, w, mom, g0, eps, L)
        H1 = _hamiltonian64(orc, m, X, y, w1, m1.astype(np.float64) + 0.5 * eps * g1)
        errs.append(abs(H1 - H0))
    assert errs[0] / errs[1] == pytest.approx(4, rel=0.35)
    assert errs[1] / errs[2] == pytest.approx(4, rel=0.35)


# ----------------------------------------------------------------------------------------------
# accept / adaptation / chain (kernel_helpers.h:153-188, main.h:204-287)
# ----------------------------------------------------------------------------------------------
def test_log_acpt_is_minus_delta_hamiltonian(orc):
    m, X, y, w = _case(orc, 200, "t", seed=12)
    mom = np.random.default_rng(12).normal(0, 1, P).astype(np.float32)
    ell0, prior0, g0, _ = orc.eval_f32(m, X, y, w)
    eps, L = 3e-3, 30
    w1, m1, g1, loss1 = orc.mcmc_step(m, X, y, w, mom, g0, eps, L)
    la = orc.log_acpt(np.concatenate([ell0, prior0]), loss1, mom, m1, g1, eps)
    H0 = _hamiltonian64(orc, m, X, y, w, mom)
    H1 = _hamiltonian64(orc, m, X, y, w1, m1.astype(np.float64) + 0.5 * eps * g1)
    assert la == pytest.approx(H0 - H1, abs=2e-4)
    assert abs(la) > 1e-3  # the test has teeth: the value is not trivially zero
    # momentum term alone: no loss change, zero gradient
    z = np.zeros(P, np.float32)
    la2 = orc.log_acpt(loss1, loss1, mom, 2 * mom, z, eps)
    assert la2 == pytest.approx(0.5 * (np.sum(mom.astype(np.float64) ** 2) * (1 - 4)), rel=1e-6)


def test_accept_rule_table(orc):
    inf, nan = float("inf"), float("nan")
    assert orc.accept(-1.0, -0.5) == 1      # log u < log a
    assert orc.accept(-0.5, -0.5) == 0      # equality rejects (strict <, main.h:242)
    assert orc.accept(-0.5, -1.0) == 0
    assert orc.accept(-1.0, nan) == 0       # divergent trajectory rejects
    assert orc.accept(-1.0, -inf) == 0
    assert orc.accept(-1.0, inf) == 1
    assert orc.accept(-1e30, 0.0) == 1


def test_adaptation_policy(orc):
    h = ob.ref_hmc()
    dec = np.float32(-0.1) / (np.float32(1) + np.float32(0.1))
    lt = math.log(0.2)
    e = np.float32(0.01)
    assert orc.adapt_eps(h, e, -0.5) == np.float32(e + e * np.float32(0.01))      # above target
    assert orc.adapt_eps(h, e, 3.0) == np.float32(e + e * np.float32(0.01))       # min(., 0)
    assert orc.adapt_eps(h, e, -5.0) == np.float32(e + e * dec)                   # below target
    assert orc.adapt_eps(h, e, float("-inf")) == np.float32(e + e * dec)
    assert orc.adapt_eps(h, e, float("nan")) == np.float32(e + e * dec)           # non-finite -> reject
    assert orc.adapt_eps(h, e, np.float32(lt) - 1e-3) == np.float32(e + e * dec)
    assert orc.adapt_eps(h, e, np.float32(lt) + 1e-3) == np.float32(e + e * np.float32(0.01))
    # a scripted sequence is a product of 1.01 and 1/1.1 factors
    seq = [-9, -9, -0.1, -9, 0.3, -0.2]
    for la in seq:
        e = orc.adapt_eps(h, e, la)
    assert e == pytest.approx(0.01 * 1.01 ** 3 / 1.1 ** 3, rel=1e-6)


def test_run_chain_bookkeeping(orc):
    n = 96
    m, X, y, _ = _case(orc, n, "gauss", seed=13)
    h = ob.Hmc(8, 12, 20, 12, 1e-2, 0.2, 0.1, 0.01, 77, 5)
    out = orc.run_chain(m, h, X, y)
    T = 32
    assert out["n_accept"] == out["accept"].sum()
    assert 0 < out["n_accept"] < T  # both branches exercised
    # replay the chain from the traces with the step operator
    w = np.zeros(P, np.float32)
    ell, prior, g, _ = orc.eval_f32(m, X, y, w)
    loss = np.concatenate([ell, prior])
    eps = np.float32(h.eps0)
    for t in range(T):
        mom = orc.momentum(77, 5, t, P)
        w1, m1, g1, loss1 = orc.mcmc_step(m, X, y, w, mom, g, float(eps), 8)
        la = orc.log_acpt(loss, loss1, mom, m1, g1, float(eps))
        assert la == out["log_acpt"][t] or (math.isnan(la) and math.isnan(out["log_acpt"][t]))
        acc = orc.accept(orc.log_uniform(77, 5, t), la)
        assert acc == out["accept"][t]
        if acc:
            w, g, loss = w1, g1, loss1
        if t < h.adapt_steps:
            eps = np.float32(orc.adapt_eps(h, float(eps), la))
        assert eps == out["eps"][t]
        if t >= h.burn_in:
            # rejected transitions duplicate the previous row (main.h:277-283)
            np.testing.assert_array_equal(out["samples"][t - h.burn_in], w)
    np.testing.assert_array_equal(out["final_w"], w)
    assert out["final_eps"] == out["eps"][h.adapt_steps - 1] == out["eps"][-1]


def test_run_chain_from_a_saved_state_is_the_tail_of_the_whole_chain(orc):
    n = 96
    m, X, y, _ = _case(orc, n, "gauss", seed=13)
    h = ob.Hmc(8, 12, 20, 12, 1e-2, 0.2, 0.1, 0.01, 77, 5)
    whole = orc.run_chain(m, h, X, y)
    for cut in (5, 12, 19):    # inside the adaptation window, at its end, among the kept samples
        head = orc.run_chain_from(m, h, X, y, None, h.eps0, 0, cut)
        assert head["accept"].tobytes() == whole["accept"][:cut].tobytes()
        tail = orc.run_chain_from(m, h, X, y, head["final_w"], head["final_eps"], cut, 32 - cut)
        assert tail["accept"].tobytes() == whole["accept"][cut:].tobytes()
        assert tail["eps"].tobytes() == whole["eps"][cut:].tobytes()
        assert tail["log_acpt"].tobytes() == whole["log_acpt"][cut:].tobytes()
        first = max(cut, h.burn_in) - h.burn_in
        assert tail["samples"][first:].tobytes() == whole["samples"][first:].tobytes()
        assert tail["final_w"].tobytes() == whole["final_w"].tobytes()


def test_row_parallel_evaluation_does_not_depend_on_the_thread_count(orc):
    n = 5000   # five chunks of 1024 rows, the last one short
    m, X, y, w = _case(orc, n, "t", seed=15)
    outs = []
    for threads in (1, 3, 8):
        orc.set_threads(threads)
        ell, prior, g, yh = orc.eval_f32(m, X, y, w)
        outs.append(ell.tobytes() + prior.tobytes() + g.tobytes() + yh.tobytes())
    orc.set_threads(8)
    assert outs[0] == outs[1] == outs[2]
    # and the chunked sum is the plain sum over rows: float64 gradient of the same model
    _, _, g64 = orc.eval_f64(m, X, y, w.astype(np.float64))
    np.testing.assert_allclose(g, g64, rtol=0, atol=2e-6 * np.abs(g64).max())


def test_cut_short_trajectories_decide_like_full_length_ones(orc):
    # the stiff Gaussian posterior with eps0 = 0.01 overflows within a few steps until the adaptation
    # has shrunk the step size: integrating on through NaN (as the reference does) and stopping at the
    # first non-finite position must give the same decisions and step sizes
    n = 512
    m, X, y, _ = _case(orc, n, "gauss", seed=16)
    h = ob.Hmc(30, 60, 4, 60, 1e-2, 0.2, 0.1, 0.01, 3, 0)
    try:
        orc.set_cut_short(False)
        full = orc.run_chain(m, h, X, y)
    finally:
        orc.set_cut_short(True)
    cut = orc.run_chain(m, h, X, y)
    assert not np.isfinite(full["log_acpt"][0]) and full["accept"][0] == 0
    assert 0 < full["accept"].sum()                      # the chain does get going
    assert cut["accept"].tobytes() == full["accept"].tobytes()
    assert cut["eps"].tobytes() == full["eps"].tobytes()
    assert cut["samples"].tobytes() == full["samples"].tobytes()
    finite = np.isfinite(full["log_acpt"])
    assert np.array_equal(finite, np.isfinite(cut["log_acpt"]))
    assert cut["log_acpt"][finite].tobytes() == full["log_acpt"][finite].tobytes()


def test_final_loss_is_mean_over_samples(orc):
    n = 50
    m, X, y, w = _case(orc, n, "t", seed=14)
    rng = np.random.default_rng(14)
    samples = (w[None, :] + rng.normal(0, 0.01, (5, P))).astype(np.float32)
    l1, l2, fl = orc.final_loss(m, X, y, samples)
    e1, e2 = [], []
    for s in samples:
        ell, prior, _, _ = orc.eval_f32(m, X, y, s)
        e1.append(ell.sum(dtype=np.float64))
        e2.append(prior.sum(dtype=np.float64))
    assert l1 == pytest.approx(np.mean(e1), rel=1e-6)
    assert l2 == pytest.approx(np.mean(e2), rel=1e-6)
    assert fl == pytest.approx(np.mean(e1) + np.mean(e2), rel=1e-6)


# ----------------------------------------------------------------------------------------------
# synthetic data generator (build-defined)
# ----------------------------------------------------------------------------------------------
def test_gen_window_recipe(orc):
    n = 4096
    X, y, th = orc.gen_window(0, 3, n)
    assert abs(X.mean()) < 4 / math.sqrt(X.size) and abs(X.var() - 1) < 0.02
    assert abs(th.std() - 0.1) < 0.01
    yh, b2, _ = _numpy_forward(X, th.astype(np.float64))
    resid = y - (yh + b2)
    assert abs(resid.std() - 0.01) < 0.001 and abs(resid.mean()) < 0.001
    # element (i, k) of X is normal(stream X, index i*d0 + k) under key (seed, window)
    assert X[7, 3] == orc.normal(0, 3, ob.STREAM_X, 0, 7 * D0 + 3)
    assert th[100] == np.float32(0.1) * np.float32(orc.normal(0, 3, ob.STREAM_TEACHER, 0, 100))
    X2, y2, _ = orc.gen_window(0, 4, 64)
    assert not np.array_equal(X2, X[:64])
    X3, y3, _ = orc.gen_window(0, 3, 64)
    assert np.array_equal(X3, X[:64]) and np.array_equal(y3, y[:64])
