"""ctypes binding of libbnn_hmc.so, the MI355X HMC sampler for the Bayesian 2-layer MLP.

The package directory name contains hyphens, so it is loaded by path (see `load_package` in
__graft_entry__.py) rather than with an import statement.  Everything here is a thin mirror of
include/bnn_hmc.h: no computation happens in Python, and there is no CPU fallback -- if the shared
library is missing or no gfx950 device is visible the calls fail.
"""
import ctypes as C
import os
import subprocess

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
LIB_PATH = os.path.join(PKG_DIR, "libbnn_hmc.so")

OK, ERR_INVALID, ERR_HIP, ERR_NO_DEVICE, ERR_RESIDENCY, ERR_TIMEOUT, ERR_STATE, ERR_DIVERGED = range(8)
LIK_STUDENT_T, LIK_GAUSSIAN = 0, 1
LAYER_MFMA, LAYER_FFMA = 0, 1
STREAM_X, STREAM_TEACHER, STREAM_NOISE, STREAM_MOMENTUM, STREAM_ACCEPT = range(5)


class Model(C.Structure):
    _fields_ = [("d0", C.c_int), ("d1", C.c_int), ("n", C.c_int), ("lik_kind", C.c_int),
                ("lik_scale", C.c_double), ("lik_df", C.c_double), ("prior_scale", C.c_double)]


class Hmc(C.Structure):
    _fields_ = [("leapfrog_steps", C.c_int), ("burn_in", C.c_int), ("n_samples", C.c_int),
                ("adapt_steps", C.c_int), ("eps0", C.c_float), ("target_rate", C.c_float),
                ("decrement", C.c_float), ("increment", C.c_float), ("seed", C.c_uint32),
                ("chain_id_base", C.c_uint32)]


class Launch(C.Structure):
    _fields_ = [("layer", C.c_int), ("cus_per_chain", C.c_int), ("wgs_per_cu", C.c_int),
                ("threads", C.c_int), ("pipeline", C.c_int),
                ("transitions_per_launch", C.c_int), ("spin_limit", C.c_uint)]


class BnnHmcError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("bnnhmc error %d: %s" % (code, msg))
        self.code = code


# every symbol include/bnn_hmc.h declares
EXPORTS = [
    "bnnhmc_default_model", "bnnhmc_default_hmc", "bnnhmc_default_launch", "bnnhmc_num_params",
    "bnnhmc_last_error", "bnnhmc_device_info", "bnnhmc_step_workspace_bytes", "bnnhmc_mcmc_step",
    "bnnhmc_mcmc_step_static", "bnnhmc_step_check", "bnnhmc_sample_momentum", "bnnhmc_log_acpt", "bnnhmc_get_loss_values",
    "bnnhmc_create", "bnnhmc_destroy", "bnnhmc_set_window_data", "bnnhmc_generate_window",
    "bnnhmc_generate_window_host", "bnnhmc_rng_word", "bnnhmc_rng_normal", "bnnhmc_rng_log_uniform",
    "bnnhmc_get_window_data", "bnnhmc_init_chains", "bnnhmc_run", "bnnhmc_get_samples",
    "bnnhmc_get_chain_state", "bnnhmc_get_traces", "bnnhmc_eval", "bnnhmc_final_loss",
    "bnnhmc_get_timing", "bnnhmc_read_reference_data", "bnnhmc_set_chain_state",
    "bnnhmc_split_rhat_ess", "bnnhmc_window_diagnostics", "bnnhmc_step_launch_info",
    "bnnhmc_get_batching",
]


def build(verbose=False):
    """Compile the HIP library for gfx950 (cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", PKG_DIR, "libbnn_hmc.so", "bnn_hmc_main"] + ([] if verbose else ["-s"]),
                   check=True)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _vp(ptr):
    return C.c_void_p(int(ptr))


class Lib:
    def __init__(self, path=LIB_PATH):
        if not os.path.exists(path):
            raise FileNotFoundError(
                "%s not built: run `python -c 'import __graft_entry__ as g; g.build()'`" % path)
        self.path = path
        self.c = C.CDLL(path)
        c = self.c
        c.bnnhmc_last_error.restype = C.c_char_p
        c.bnnhmc_num_params.restype = C.c_int
        c.bnnhmc_step_workspace_bytes.restype = C.c_size_t
        c.bnnhmc_rng_word.restype = C.c_uint32
        c.bnnhmc_rng_word.argtypes = [C.c_uint32] * 4 + [C.c_uint64]
        c.bnnhmc_rng_normal.restype = C.c_float
        c.bnnhmc_rng_normal.argtypes = [C.c_uint32] * 4 + [C.c_uint64]
        c.bnnhmc_rng_log_uniform.restype = C.c_float
        c.bnnhmc_rng_log_uniform.argtypes = [C.c_uint32] * 3

    # ---- helpers ----
    def check(self, rc):
        if rc != OK:
            raise BnnHmcError(rc, self.c.bnnhmc_last_error().decode())

    def default_model(self, **kw):
        m = Model()
        self.c.bnnhmc_default_model(C.byref(m))
        for k, v in kw.items():
            setattr(m, k, v)
        return m

    def default_hmc(self, **kw):
        h = Hmc()
        self.c.bnnhmc_default_hmc(C.byref(h))
        for k, v in kw.items():
            setattr(h, k, v)
        if "burn_in" in kw and "adapt_steps" not in kw:
            h.adapt_steps = h.burn_in
        return h

    def default_launch(self, **kw):
        l = Launch()
        self.c.bnnhmc_default_launch(C.byref(l))
        for k, v in kw.items():
            setattr(l, k, v)
        return l

    def num_params(self, d0, d1):
        return self.c.bnnhmc_num_params(d0, d1)

    def device_info(self):
        n, cus = C.c_int(), C.c_int()
        arch = C.create_string_buffer(64)
        rc = self.c.bnnhmc_device_info(C.byref(n), C.byref(cus), arch, C.c_size_t(64))
        return rc, n.value, cus.value, arch.value.decode()

    # ---- host-only pieces ----
    def generate_window_host(self, seed, window, n, d0=22, d1=40, teacher_scale=0.1, noise_sigma=0.01):
        P = self.num_params(d0, d1)
        X = np.empty((n, d0), np.float32)
        y = np.empty(n, np.float32)
        th = np.empty(P, np.float32)
        self.check(self.c.bnnhmc_generate_window_host(
            C.c_uint32(seed), C.c_uint32(window), C.c_int(n), C.c_int(d0), C.c_int(d1),
            C.c_float(teacher_scale), C.c_float(noise_sigma), _fp(X), _fp(y), _fp(th)))
        return X, y, th

    def read_reference_data(self, path, n, d0=22, total_cols=149, skip_cols=2):
        X = np.empty((n, d0), np.float32)
        y = np.empty(n, np.float32)
        self.check(self.c.bnnhmc_read_reference_data(path.encode(), C.c_int(n), C.c_int(d0),
                                                     C.c_int(total_cols), C.c_int(skip_cols), _fp(X), _fp(y)))
        return X, y

    def split_rhat_ess(self, samples):
        """samples[chain][draw][param] (float32, host) -> (split R-hat, effective sample size)."""
        x = np.ascontiguousarray(samples, np.float32)
        assert x.ndim == 3
        nc, ns, npar = x.shape
        rhat = np.empty(npar, np.float64)
        ess = np.empty(npar, np.float64)
        self.check(self.c.bnnhmc_split_rhat_ess(_fp(x), C.c_int(nc), C.c_int(ns), C.c_int(npar),
                                                C.c_size_t(ns * npar), rhat.ctypes.data_as(C.c_void_p),
                                                ess.ctypes.data_as(C.c_void_p)))
        return rhat, ess

    def rng_word(self, seed, id_, stream, t, index):
        return self.c.bnnhmc_rng_word(seed, id_, stream, t, index)

    def rng_normal(self, seed, id_, stream, t, index):
        return self.c.bnnhmc_rng_normal(seed, id_, stream, t, index)

    def rng_log_uniform(self, seed, chain, t):
        return self.c.bnnhmc_rng_log_uniform(seed, chain, t)

    # ---- operator level (device pointers given as integers) ----
    def step_workspace_bytes(self, model, launch):
        return self.c.bnnhmc_step_workspace_bytes(C.byref(model), C.byref(launch))

    def mcmc_step(self, model, launch, x, y, w_prev, w_next, m_prev, m_next, g_prev, g_cur, g_next,
                  loss, workspace, workspace_bytes, eps, lp_steps, stream=0):
        self.check(self.c.bnnhmc_mcmc_step(
            C.byref(model), C.byref(launch), _vp(x), _vp(y), _vp(w_prev), _vp(w_next), _vp(m_prev),
            _vp(m_next), _vp(g_prev), _vp(g_cur), _vp(g_next), _vp(loss), _vp(workspace),
            C.c_size_t(workspace_bytes), C.c_float(eps), C.c_int(lp_steps), _vp(stream)))

    def mcmc_step_static(self, model, launch, x, y, w_prev, w_next, m_prev, m_next, g_prev, g_cur, g_next,
                         loss, eps, lp_steps, stream=0):
        self.check(self.c.bnnhmc_mcmc_step_static(
            C.byref(model), C.byref(launch), _vp(x), _vp(y), _vp(w_prev), _vp(w_next), _vp(m_prev),
            _vp(m_next), _vp(g_prev), _vp(g_cur), _vp(g_next), _vp(loss), C.c_float(eps),
            C.c_int(lp_steps), _vp(stream)))

    def step_check(self, model, launch, workspace, stream=0):
        self.check(self.c.bnnhmc_step_check(C.byref(model), C.byref(launch), _vp(workspace), _vp(stream)))

    def sample_momentum(self, seed, chain, t, n, a, b, stream=0):
        self.check(self.c.bnnhmc_sample_momentum(C.c_uint32(seed), C.c_uint32(chain), C.c_uint32(t),
                                                 C.c_int(n), _vp(a), _vp(b), _vp(stream)))

    def log_acpt(self, n_loss, n_mom, prev_loss, new_loss, prev_mom, new_mom, grad_cur, eps, out_dev,
                 stream=0):
        h = C.c_float()
        self.check(self.c.bnnhmc_log_acpt(C.c_int(n_loss), C.c_int(n_mom), _vp(prev_loss), _vp(new_loss),
                                          _vp(prev_mom), _vp(new_mom), _vp(grad_cur), C.c_float(eps),
                                          _vp(out_dev), C.byref(h), _vp(stream)))
        return h.value

    def get_loss_values(self, loss, n, n_params, stream=0):
        a, b = C.c_float(), C.c_float()
        self.check(self.c.bnnhmc_get_loss_values(_vp(loss), C.c_int(n), C.c_int(n_params), C.byref(a),
                                                 C.byref(b), _vp(stream)))
        return a.value, b.value

    # ---- sampler level ----
    def create(self, model, hmc, launch, n_windows=1, chains_per_window=1):
        return Sampler(self, model, hmc, launch, n_windows, chains_per_window)


class Sampler:
    """Owns a bnnhmc_sampler handle: init (create / data / init_chains), run, dump."""

    def __init__(self, lib, model, hmc, launch, n_windows, chains_per_window):
        self.lib = lib
        self.model, self.hmc, self.launch = model, hmc, launch
        self.n_windows, self.cpw = n_windows, chains_per_window
        self.P = lib.num_params(model.d0, model.d1)
        self.h = C.c_void_p()
        lib.check(lib.c.bnnhmc_create(C.byref(model), C.byref(hmc), C.byref(launch), C.c_int(n_windows),
                                      C.c_int(chains_per_window), C.byref(self.h)))

    def close(self):
        if self.h:
            self.lib.c.bnnhmc_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_window_data(self, window, X, y):
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        assert X.shape == (self.model.n, self.model.d0) and y.shape == (self.model.n,)
        self.lib.check(self.lib.c.bnnhmc_set_window_data(self.h, C.c_int(window), _fp(X), _fp(y)))

    def generate_window(self, window, teacher_scale=0.1, noise_sigma=0.01):
        th = np.empty(self.P, np.float32)
        self.lib.check(self.lib.c.bnnhmc_generate_window(self.h, C.c_int(window), C.c_float(teacher_scale),
                                                         C.c_float(noise_sigma), _fp(th)))
        return th

    def get_window_data(self, window):
        X = np.empty((self.model.n, self.model.d0), np.float32)
        y = np.empty(self.model.n, np.float32)
        self.lib.check(self.lib.c.bnnhmc_get_window_data(self.h, C.c_int(window), _fp(X), _fp(y)))
        return X, y

    def init_chains(self, w0=None):
        if w0 is None:
            self.lib.check(self.lib.c.bnnhmc_init_chains(self.h, None))
        else:
            w0 = np.ascontiguousarray(w0, np.float32)
            assert w0.shape == (self.P,)
            self.lib.check(self.lib.c.bnnhmc_init_chains(self.h, _fp(w0)))

    def run(self, n_transitions):
        self.lib.check(self.lib.c.bnnhmc_run(self.h, C.c_int(n_transitions)))

    def get_samples(self, chain):
        out = np.empty((self.hmc.n_samples, self.P), np.float32)
        n = C.c_int()
        self.lib.check(self.lib.c.bnnhmc_get_samples(self.h, C.c_int(chain), _fp(out), C.byref(n)))
        return out[:n.value]

    def get_chain_state(self, chain):
        w = np.empty(self.P, np.float32)
        g = np.empty(self.P, np.float32)
        eps, t, na = C.c_float(), C.c_int(), C.c_int()
        self.lib.check(self.lib.c.bnnhmc_get_chain_state(self.h, C.c_int(chain), _fp(w), _fp(g),
                                                         C.byref(eps), C.byref(t), C.byref(na)))
        return dict(w=w, grad=g, eps=eps.value, transitions_done=t.value, n_accepted=na.value)

    def set_chain_state(self, chain, w, eps, transitions_done, n_accepted):
        w = np.ascontiguousarray(w, np.float32)
        assert w.shape == (self.P,)
        self.lib.check(self.lib.c.bnnhmc_set_chain_state(self.h, C.c_int(chain), _fp(w), C.c_float(eps),
                                                         C.c_int(transitions_done), C.c_int(n_accepted)))

    def get_traces(self, chain):
        T = self.hmc.burn_in + self.hmc.n_samples
        la = np.full(T, np.nan, np.float32)
        acc = np.full(T, -1, np.int32)
        eps = np.full(T, np.nan, np.float32)
        self.lib.check(self.lib.c.bnnhmc_get_traces(self.h, C.c_int(chain), _fp(la),
                                                    acc.ctypes.data_as(C.POINTER(C.c_int)), _fp(eps)))
        done = self.get_chain_state(chain)["transitions_done"]
        n = min(done, T)
        return dict(log_acpt=la[:n], accept=acc[:n], eps=eps[:n])

    def eval(self, window, w):
        w = np.ascontiguousarray(w, np.float32)
        assert w.shape == (self.P,)
        ell = np.empty(self.model.n, np.float32)
        prior = np.empty(self.P, np.float32)
        grad = np.empty(self.P, np.float32)
        self.lib.check(self.lib.c.bnnhmc_eval(self.h, C.c_int(window), _fp(w), _fp(ell), _fp(prior),
                                              _fp(grad)))
        return ell, prior, grad

    def final_loss(self, chain):
        a, b, c = C.c_double(), C.c_double(), C.c_double()
        self.lib.check(self.lib.c.bnnhmc_final_loss(self.h, C.c_int(chain), C.byref(a), C.byref(b),
                                                    C.byref(c)))
        return a.value, b.value, c.value

    def diagnostics(self, window):
        """(split R-hat, effective sample size) per parameter over the chains of a window."""
        rhat = np.empty(self.P, np.float64)
        ess = np.empty(self.P, np.float64)
        self.lib.check(self.lib.c.bnnhmc_window_diagnostics(
            self.h, window, rhat.ctypes.data_as(C.c_void_p), ess.ctypes.data_as(C.c_void_p)))
        return rhat, ess

    def batching(self):
        """(chains in a full launch, workgroups per chain in it)"""
        b, g = C.c_int(), C.c_int()
        self.lib.check(self.lib.c.bnnhmc_get_batching(self.h, C.byref(b), C.byref(g), None))
        return b.value, g.value

    def batch_trial_rates(self):
        """gradient evaluations/s of the last timed pair of launches: (the shape within the row budget, the device-wide shape)"""
        r = (C.c_double * 2)()
        self.lib.check(self.lib.c.bnnhmc_get_batching(self.h, None, None, r))
        return r[0], r[1]

    def timing(self):
        ms, launches, evals, wgs = C.c_double(), C.c_long(), C.c_long(), C.c_int()
        self.lib.check(self.lib.c.bnnhmc_get_timing(self.h, C.byref(ms), C.byref(launches),
                                                    C.byref(evals), C.byref(wgs)))
        return dict(kernel_ms=ms.value, launches=launches.value, grad_evals=evals.value,
                    workgroups=wgs.value)


_LIB = None


def load():
    """The loaded library (fails loudly if it has not been built)."""
    global _LIB
    if _LIB is None:
        _LIB = Lib()
    return _LIB
