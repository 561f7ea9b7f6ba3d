"""CPU-only checks of the shipped library: it loads, exports the whole C ABI, its host-side
generator and RNG agree bit for bit with the oracle's independent restatement, and its error paths
return codes instead of aborting.  No compute is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import orc_binding as ob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(pkg, lib):
    header = open(os.path.join(ROOT, "include", "bnn_hmc.h")).read()
    declared = set(re.findall(r"\b(bnnhmc_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(pkg.EXPORTS)
    for name in declared:
        assert hasattr(lib.c, name), name


def test_struct_layouts_match_header(pkg):
    assert C.sizeof(pkg.Model) == 4 * 4 + 3 * 8
    assert C.sizeof(pkg.Hmc) == 4 * 4 + 4 * 4 + 2 * 4
    assert C.sizeof(pkg.Launch) == 7 * 4


def test_defaults_are_the_reference_constants(lib):
    m = lib.default_model()
    assert (m.d0, m.d1, m.n) == (22, 40, 58368)                      # global_params.h:56, 61
    assert (m.lik_kind, m.lik_scale, m.lik_df, m.prior_scale) == (0, 100.0, 2.2, 200.0)
    h = lib.default_hmc()
    assert (h.leapfrog_steps, h.burn_in, h.n_samples, h.adapt_steps) == (1000, 100, 800, 100)
    assert h.eps0 == np.float32(0.01) and h.target_rate == np.float32(0.2)
    assert h.decrement == np.float32(0.1) and h.increment == np.float32(0.01)
    assert lib.num_params(22, 40) == 961


def test_host_rng_matches_oracle_bit_for_bit(lib, orc):
    for (seed, id_, stream, t, idx) in [(0, 0, 3, 0, 0), (7, 199, 3, 899, 960), (1, 2, 0, 0, 1284095),
                                        (123456789, 799, 4, 1699, 0), (5, 6, 2, 0, 58367)]:
        assert lib.rng_word(seed, id_, stream, t, idx) == orc.rng_word(seed, id_, stream, t, idx)
        a = np.float32(lib.rng_normal(seed, id_, stream, t, idx))
        b = np.float32(orc.normal(seed, id_, stream, t, idx))
        assert a.tobytes() == b.tobytes()
    for t in range(200):
        a = np.float32(lib.rng_log_uniform(3, 4, t))
        b = np.float32(orc.log_uniform(3, 4, t))
        assert a.tobytes() == b.tobytes()
    mom = orc.momentum(11, 5, 17, 961)
    mine = np.array([lib.rng_normal(11, 5, 3, 17, p) for p in range(961)], np.float32)
    assert mine.tobytes() == mom.tobytes()


def test_host_generator_matches_oracle_bit_for_bit(lib, orc):
    for (seed, window, n) in [(0, 0, 300), (0, 7, 64), (9, 199, 33)]:
        X, y, th = lib.generate_window_host(seed, window, n)
        Xo, yo, tho = orc.gen_window(seed, window, n)
        assert X.tobytes() == Xo.tobytes()
        assert th.tobytes() == tho.tobytes()
        assert y.tobytes() == yo.tobytes()


def test_error_codes_without_launching(pkg, lib):
    m = lib.default_model()
    h = lib.default_hmc()
    l = lib.default_launch()
    hnd = C.c_void_p()
    # unsupported shape
    bad = lib.default_model(d0=23)
    rc = lib.c.bnnhmc_create(C.byref(bad), C.byref(h), C.byref(l), 1, 1, C.byref(hnd))
    assert rc == pkg.ERR_INVALID and b"unsupported layer sizes" in lib.c.bnnhmc_last_error()
    for kw in (dict(n=0), dict(lik_kind=5), dict(lik_scale=0.0), dict(prior_scale=-1.0), dict(lik_df=0.0)):
        bad = lib.default_model(**kw)
        assert lib.c.bnnhmc_create(C.byref(bad), C.byref(h), C.byref(l), 1, 1, C.byref(hnd)) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_create(None, C.byref(h), C.byref(l), 1, 1, C.byref(hnd)) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_create(C.byref(m), None, C.byref(l), 1, 1, C.byref(hnd)) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_create(C.byref(m), C.byref(h), C.byref(l), 0, 1, C.byref(hnd)) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_create(C.byref(m), C.byref(h), C.byref(l), 1, 1, None) == pkg.ERR_INVALID
    badh = lib.default_hmc(leapfrog_steps=0)
    assert lib.c.bnnhmc_create(C.byref(m), C.byref(badh), C.byref(l), 1, 1, C.byref(hnd)) == pkg.ERR_INVALID
    # null handles
    assert lib.c.bnnhmc_run(None, 1) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_init_chains(None, None) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_get_samples(None, 0, None, None) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_destroy(None) == pkg.OK
    # operator level: null pointers and bad sizes are rejected before anything is launched
    rc = lib.c.bnnhmc_mcmc_step(C.byref(m), C.byref(l), None, None, None, None, None, None, None, None,
                                None, None, None, C.c_size_t(0), C.c_float(0.01), 1, None)
    assert rc == pkg.ERR_INVALID
    assert lib.c.bnnhmc_log_acpt(-1, 0, None, None, None, None, None, C.c_float(0), None, None, None) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_sample_momentum(0, 0, 0, -1, None, None, None) == pkg.ERR_INVALID
    assert lib.c.bnnhmc_get_loss_values(None, 1, 1, None, None, None) == pkg.ERR_INVALID
    assert lib.step_workspace_bytes(m, l) >= 2 * 256 * 961 * 4


def test_no_device_is_reported_not_faked(pkg, lib):
    rc, n_dev, cus, arch = lib.device_info()
    if n_dev > 0:
        pytest.skip("a GPU is visible")
    assert rc == pkg.ERR_NO_DEVICE
    m, h, l = lib.default_model(n=64), lib.default_hmc(), lib.default_launch()
    hnd = C.c_void_p()
    assert lib.c.bnnhmc_create(C.byref(m), C.byref(h), C.byref(l), 1, 1, C.byref(hnd)) == pkg.ERR_NO_DEVICE
    assert not hnd.value


def test_reference_text_reader(lib, pkg, tmp_path):
    # the reference's file layout (io.h:43-86): header line, then 149 columns per row of which the
    # first 2 are skipped, column 2 is the label and columns 3..24 are the 22 features
    rng = np.random.default_rng(0)
    n, cols = 7, 149
    table = rng.normal(0, 3, (n, cols)).round(4)
    path = tmp_path / "returns_and_features_for_mcmc.txt"
    with open(path, "w") as f:
        f.write(" ".join("col%d" % j for j in range(cols)) + "\n")
        for i in range(n):
            f.write(" ".join(["2020-01-%02d" % (i + 1), "ID%d" % i] + ["%.4f" % v for v in table[i, 2:]]) + "\n")
    X, y = lib.read_reference_data(str(path), n)
    np.testing.assert_array_equal(y, table[:, 2].astype(np.float32))
    np.testing.assert_array_equal(X, table[:, 3:25].astype(np.float32))
    # a short file and a missing file are errors, not aborts
    with pytest.raises(pkg.BnnHmcError) as e:
        lib.read_reference_data(str(path), n + 1)
    assert e.value.code == pkg.ERR_INVALID and "ends at row" in str(e.value)
    with pytest.raises(pkg.BnnHmcError):
        lib.read_reference_data(str(tmp_path / "missing.txt"), n)


# ------------------------------------------------------------------------------------------------
# convergence diagnostics (host arithmetic, no GPU)
# ------------------------------------------------------------------------------------------------
def _numpy_split_rhat_ess(x):
    """The estimators of Vehtari et al. 2021 (no rank normalisation) written independently with numpy:
    autocovariances by FFT, Geyer's initial positive sequence with the monotone correction."""
    nc, ns, _ = x.shape
    n = ns // 2
    seq = np.concatenate([x[:, :n], x[:, ns - n:]], axis=0).astype(np.float64)  # order differs: harmless
    m = seq.shape[0]
    mean = seq.mean(axis=1)
    var = seq.var(axis=1, ddof=1)
    W = var.mean(axis=0)
    var_plus = (n - 1) / n * W + mean.var(axis=0, ddof=1)
    rhat = np.sqrt(var_plus / W)
    ess = np.empty(x.shape[2])
    for p in range(x.shape[2]):
        c = seq[:, :, p] - mean[:, None, p]
        f = np.fft.rfft(c, 2 * n, axis=1)
        acov = np.fft.irfft(f * np.conj(f), 2 * n, axis=1)[:, :n] / (n - 1)
        rho = 1.0 - (W[p] - acov.mean(axis=0)) / var_plus[p]
        tau, prev = -1.0, None
        for t in range(0, n - 1, 2):
            pair = rho[t] + rho[t + 1]
            if not pair > 0:
                break
            if prev is not None and pair > prev:
                pair = prev
            tau += 2 * pair
            prev = pair
        tau = max(tau, 1 / np.log10(m * n))
        ess[p] = m * n / tau
    return rhat, ess


def test_split_rhat_and_ess(lib, pkg):
    rng = np.random.default_rng(12)
    C_, S, Pn = 4, 800, 6
    phi = np.array([0.0, 0.5, 0.9, -0.5, 0.0, 0.0])
    x = np.empty((C_, S, Pn), np.float64)
    e = rng.normal(size=(C_, S + 200, Pn))
    z = np.zeros((C_, Pn))
    out = []
    for t in range(S + 200):                      # stationary AR(1) with unit marginal variance
        z = phi * z + np.sqrt(1 - phi ** 2) * e[:, t]
        out.append(z.copy())
    x[:] = np.stack(out[200:], axis=1)
    x[:, :, 4] += np.array([0.0, 0.0, 0.0, 3.0])[:, None]     # one chain sits elsewhere
    x[:, :, 5] = 1.25                                          # a parameter that never moves
    xs = x.astype(np.float32)
    rhat, ess = lib.split_rhat_ess(xs)
    # against an independent numpy / FFT implementation of the same published estimators
    r_np, e_np = _numpy_split_rhat_ess(xs[:, :, :5])
    np.testing.assert_allclose(rhat[:5], r_np, rtol=1e-9)
    np.testing.assert_allclose(ess[:5], e_np, rtol=1e-6)
    # against what the processes fix: iid draws ~ all 3200 count, AR(1) keeps N (1 - phi) / (1 + phi)
    N = C_ * S
    assert 0.8 * N < ess[0] < 1.2 * N and rhat[0] < 1.01
    assert ess[1] == pytest.approx(N / 3, rel=0.25) and rhat[1] < 1.02
    assert ess[2] == pytest.approx(N / 19, rel=0.4) and rhat[2] < 1.1
    assert ess[3] > 1.5 * N                                    # antithetic draws beat iid
    assert rhat[4] > 1.5 and ess[4] < 20                       # disagreeing chains are flagged
    assert rhat[5] == 1.0 and ess[5] == N                      # constant parameter
    # one chain only: split halves still work
    r1, e1 = lib.split_rhat_ess(xs[:1])
    assert r1[0] < 1.02 and 0.6 * S < e1[0] < 1.4 * S
    with pytest.raises(pkg.BnnHmcError):
        lib.split_rhat_ess(xs[:, :7])


def test_step_workspace_holds_what_the_exchange_needs(lib):
    """Sizes from bnnhmc_step_workspace_bytes against what the exchange of the 22 -> 40 -> 1 kernel must
    hold whatever its layout: two records (double buffer) of P eight-byte packets per workgroup, and
    from 32 workgroups on at least one more such record for the totals; never less for more workgroups;
    and every single-chain configuration up to 256 workgroups fits the 4.5 MiB static scratch of
    bnnhmc_mcmc_step_static."""
    m = lib.default_model()
    P = lib.c.bnnhmc_num_params(m.d0, m.d1)
    prev = 0
    for G in (1, 2, 4, 8, 16, 32, 64, 128, 256):
        launch = lib.default_launch(cus_per_chain=G)
        n = lib.c.bnnhmc_step_workspace_bytes(C.byref(m), C.byref(launch))
        need = 2 * G * P * 8 + (P * 8 if G >= 32 else 0) + 64 * 4
        assert n >= need, (G, n, need)
        assert n % 16 == 0 and n >= prev
        assert n <= 4608 * 1024
        prev = n
    # the default of the step operator is the widest group
    assert lib.c.bnnhmc_step_workspace_bytes(C.byref(m), C.byref(lib.default_launch())) == prev


def test_operator_header_compiles_with_the_host_compiler(pkg, tmp_path):
    """include/mcmc_step_hip.h offers what the reference's driver takes from its operator header
    (main.h:38-42, 52-59, 120-133; mcmc_step_ffma.h:46-70, 395-436).  Compiled here by g++ against
    stand-ins for the reference's constants and its DeviceMatrix (driver/shim_check.cpp), linked against
    the library; without a GPU the program stops at its device check."""
    import subprocess

    header = open(os.path.join(ROOT, "include", "mcmc_step_hip.h")).read()
    for name in ("set_dynamic_smem_max_size", "full_smem_size", "leapfrog_max_smem_size", "N_WARP_SAMPLES",
                 "N_BLKS", "N_BLK_SAMPLES", "N_THREADS", "N_P_ALIGNED", "void mcmc_step("):
        assert name in header, name
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    exe = tmp_path / "shim_check"
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(rocm, "include"), "-o", str(exe),
           os.path.join(pkg.PKG_DIR, "driver", "shim_check.cpp"), "-L" + pkg.PKG_DIR, "-lbnn_hmc",
           "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + pkg.PKG_DIR,
           "-Wl,-rpath," + os.path.join(rocm, "lib")]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert r.returncode in (0, 3), r.stdout + r.stderr
    if r.returncode == 3:
        assert "no HIP device" in r.stderr
    # the copy built with the library is there too (the GPU test runs that one)
    assert os.path.exists(os.path.join(pkg.PKG_DIR, "shim_check"))


def test_flag_counter_bound_is_checked_on_the_host(pkg, lib):
    # the exchange numbers the leapfrog steps of a launch in 32 bits: refused before any device work
    h = lib.default_hmc(leapfrog_steps=2 ** 30)
    l = lib.default_launch(transitions_per_launch=8)
    hnd = C.c_void_p()
    rc = lib.c.bnnhmc_create(C.byref(lib.default_model()), C.byref(h), C.byref(l), 1, 1, C.byref(hnd))
    assert rc == pkg.ERR_INVALID and b"2^32" in lib.c.bnnhmc_last_error()
