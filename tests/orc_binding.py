"""ctypes binding of the CPU oracle (oracle/libbnn_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "libbnn_oracle.so")

LIK_STUDENT_T, LIK_GAUSSIAN = 0, 1
STREAM_X, STREAM_TEACHER, STREAM_NOISE, STREAM_MOMENTUM, STREAM_ACCEPT = range(5)


class Model(C.Structure):
    _fields_ = [("d0", C.c_int), ("d1", C.c_int), ("n", C.c_int), ("lik_kind", C.c_int),
                ("lik_scale", C.c_double), ("lik_df", C.c_double), ("prior_scale", C.c_double)]


class Hmc(C.Structure):
    _fields_ = [("leapfrog_steps", C.c_int), ("burn_in", C.c_int), ("n_samples", C.c_int),
                ("adapt_steps", C.c_int), ("eps0", C.c_float), ("target_rate", C.c_float),
                ("decrement", C.c_float), ("increment", C.c_float), ("seed", C.c_uint32),
                ("chain_id", C.c_uint32)]


def ref_model(n=58368, d0=22, d1=40):
    """The reference's model constants (global_params.h:39-61)."""
    return Model(d0, d1, n, LIK_STUDENT_T, 100.0, 2.2, 200.0)


def gauss_model(n=58368, d0=22, d1=40, sigma=0.01, prior=0.1):
    """The benchmark configs' Gaussian likelihood / Gaussian prior."""
    return Model(d0, d1, n, LIK_GAUSSIAN, sigma, 0.0, prior)


def ref_hmc(L=1000, burn_in=100, n_samples=800, seed=0, chain_id=0, eps0=0.01):
    return Hmc(L, burn_in, n_samples, burn_in, eps0, 0.2, 0.1, 0.01, seed, chain_id)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        L = lib
        L.orc_num_params.restype = C.c_int
        L.orc_det_log.restype = C.c_double
        L.orc_det_log.argtypes = [C.c_double]
        L.orc_det_sqrt.restype = C.c_double
        L.orc_det_sqrt.argtypes = [C.c_double]
        L.orc_ppnd16.restype = C.c_double
        L.orc_ppnd16.argtypes = [C.c_double]
        L.orc_rng_word.restype = C.c_uint32
        L.orc_rng_word.argtypes = [C.c_uint32] * 4 + [C.c_uint64]
        L.orc_normal.restype = C.c_float
        L.orc_normal.argtypes = [C.c_uint32] * 4 + [C.c_uint64]
        L.orc_log_uniform.restype = C.c_float
        L.orc_log_uniform.argtypes = [C.c_uint32] * 3
        L.orc_tanh_fwd.restype = C.c_float
        L.orc_tanh_fwd.argtypes = [C.c_float]
        L.orc_tanh_bwd.restype = C.c_float
        L.orc_tanh_bwd.argtypes = [C.c_float, C.c_float]
        L.orc_log_acpt.restype = C.c_float
        L.orc_accept.restype = C.c_int
        L.orc_accept.argtypes = [C.c_float, C.c_float]
        L.orc_adapt_eps.restype = C.c_float
        L.orc_adapt_eps.argtypes = [C.POINTER(Hmc), C.c_float, C.c_float]
        L.orc_run_chain.restype = C.c_int
        L.orc_run_chain_from.restype = C.c_int
        L.orc_bench_grad_evals.restype = C.c_double

    def set_threads(self, threads):
        self.lib.orc_set_threads(C.c_int(threads))

    def set_cut_short(self, on):
        self.lib.orc_set_cut_short(C.c_int(1 if on else 0))

    def num_params(self, d0, d1):
        return self.lib.orc_num_params(d0, d1)

    def philox(self, ctr, key):
        c = (C.c_uint32 * 4)(*ctr)
        k = (C.c_uint32 * 2)(*key)
        o = (C.c_uint32 * 4)()
        self.lib.orc_philox4x32_10(c, k, o)
        return list(o)

    def det_log(self, x):
        return self.lib.orc_det_log(x)

    def det_sqrt(self, x):
        return self.lib.orc_det_sqrt(x)

    def ppnd16(self, p):
        return self.lib.orc_ppnd16(p)

    def rng_word(self, seed, id_, stream, t, index):
        return self.lib.orc_rng_word(seed, id_, stream, t, index)

    def normal(self, seed, id_, stream, t, index):
        return self.lib.orc_normal(seed, id_, stream, t, index)

    def momentum(self, seed, chain, t, P):
        out = np.empty(P, np.float32)
        self.lib.orc_momentum(C.c_uint32(seed), C.c_uint32(chain), C.c_uint32(t), C.c_int(P), _fp(out))
        return out

    def log_uniform(self, seed, chain, t):
        return self.lib.orc_log_uniform(seed, chain, t)

    def gen_window(self, seed, window, n, d0=22, d1=40, teacher_scale=0.1, noise_sigma=0.01):
        P = self.num_params(d0, d1)
        X = np.empty((n, d0), np.float32)
        y = np.empty(n, np.float32)
        th = np.empty(P, np.float32)
        self.lib.orc_gen_window(C.c_uint32(seed), C.c_uint32(window), C.c_int(n), C.c_int(d0),
                                C.c_int(d1), C.c_float(teacher_scale), C.c_float(noise_sigma),
                                _fp(X), _fp(y), _fp(th))
        return X, y, th

    def tanh_fwd(self, x):
        return self.lib.orc_tanh_fwd(x)

    def tanh_bwd(self, out, dg):
        return self.lib.orc_tanh_bwd(out, dg)

    def row_loglik(self, m, y, yhat, b2):
        ell = C.c_float()
        g = C.c_float()
        self.lib.orc_row_loglik(C.byref(m), C.c_float(y), C.c_float(yhat), C.c_float(b2),
                                C.byref(ell), C.byref(g))
        return ell.value, g.value

    def prior_terms(self, m, w):
        lp = C.c_float()
        g = C.c_float()
        self.lib.orc_prior_terms(C.byref(m), C.c_float(w), C.byref(lp), C.byref(g))
        return lp.value, g.value

    def eval_f32(self, m, X, y, w):
        P = self.num_params(m.d0, m.d1)
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        ell = np.empty(m.n, np.float32)
        prior = np.empty(P, np.float32)
        grad = np.empty(P, np.float32)
        yhat = np.empty(m.n, np.float32)
        self.lib.orc_eval_f32(C.byref(m), _fp(X), _fp(y), _fp(w), _fp(ell), _fp(prior), _fp(grad),
                              _fp(yhat))
        return ell, prior, grad, yhat

    def eval_f64(self, m, X, y, w):
        P = self.num_params(m.d0, m.d1)
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        w = np.ascontiguousarray(w, np.float64)
        ell = np.empty(m.n, np.float64)
        prior = np.empty(P, np.float64)
        grad = np.empty(P, np.float64)
        self.lib.orc_eval_f64(C.byref(m), _fp(X), _fp(y), _dp(w), _dp(ell), _dp(prior), _dp(grad))
        return ell, prior, grad

    def mcmc_step(self, m, X, y, w_prev, mom_prev, grad_prev, eps, L):
        P = self.num_params(m.d0, m.d1)
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        w_prev = np.ascontiguousarray(w_prev, np.float32)
        mom_prev = np.ascontiguousarray(mom_prev, np.float32)
        grad_prev = np.ascontiguousarray(grad_prev, np.float32)
        w_next = np.empty(P, np.float32)
        mom_next = np.empty(P, np.float32)
        grad_cur = np.empty(P, np.float32)
        loss = np.empty(m.n + P, np.float32)
        self.lib.orc_mcmc_step(C.byref(m), _fp(X), _fp(y), _fp(w_prev), _fp(mom_prev), _fp(grad_prev),
                               C.c_float(eps), C.c_int(L), _fp(w_next), _fp(mom_next), _fp(grad_cur),
                               _fp(loss))
        return w_next, mom_next, grad_cur, loss

    def log_acpt(self, prev_loss, new_loss, prev_mom, new_mom, grad_cur, eps):
        prev_loss = np.ascontiguousarray(prev_loss, np.float32)
        new_loss = np.ascontiguousarray(new_loss, np.float32)
        prev_mom = np.ascontiguousarray(prev_mom, np.float32)
        new_mom = np.ascontiguousarray(new_mom, np.float32)
        grad_cur = np.ascontiguousarray(grad_cur, np.float32)
        return self.lib.orc_log_acpt(C.c_int(len(new_loss)), C.c_int(len(new_mom)), _fp(prev_loss),
                                     _fp(new_loss), _fp(prev_mom), _fp(new_mom), _fp(grad_cur),
                                     C.c_float(eps))

    def accept(self, log_u, log_acpt):
        return self.lib.orc_accept(log_u, log_acpt)

    def adapt_eps(self, h, eps, log_acpt):
        return self.lib.orc_adapt_eps(C.byref(h), eps, log_acpt)

    def run_chain(self, m, h, X, y):
        P = self.num_params(m.d0, m.d1)
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        T = h.burn_in + h.n_samples
        samples = np.empty((h.n_samples, P), np.float32)
        la = np.empty(T, np.float32)
        acc = np.empty(T, np.int32)
        eps = np.empty(T, np.float32)
        fw = np.empty(P, np.float32)
        fe = C.c_float()
        n_acc = self.lib.orc_run_chain(C.byref(m), C.byref(h), _fp(X), _fp(y), _fp(samples), _fp(la),
                                       acc.ctypes.data_as(C.POINTER(C.c_int)), _fp(eps), _fp(fw),
                                       C.byref(fe))
        return dict(samples=samples, log_acpt=la, accept=acc, eps=eps, final_w=fw,
                    final_eps=fe.value, n_accept=n_acc)

    def run_chain_from(self, m, h, X, y, w0, eps0, t0, n_trans):
        """n_trans transitions from position w0 (None = zeros), step size eps0, transition index t0."""
        P = self.num_params(m.d0, m.d1)
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        w0p = None if w0 is None else _fp(np.ascontiguousarray(w0, np.float32))
        samples = np.full((max(h.n_samples, 1), P), np.nan, np.float32)
        la = np.empty(n_trans, np.float32)
        acc = np.empty(n_trans, np.int32)
        eps = np.empty(n_trans, np.float32)
        fw = np.empty(P, np.float32)
        fe = C.c_float()
        n_acc = self.lib.orc_run_chain_from(C.byref(m), C.byref(h), _fp(X), _fp(y), w0p, C.c_float(eps0),
                                            C.c_int(t0), C.c_int(n_trans), _fp(samples), _fp(la),
                                            acc.ctypes.data_as(C.POINTER(C.c_int)), _fp(eps), _fp(fw),
                                            C.byref(fe))
        return dict(samples=samples[:h.n_samples], log_acpt=la, accept=acc, eps=eps, final_w=fw,
                    final_eps=fe.value, n_accept=n_acc)

    def final_loss(self, m, X, y, samples):
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        samples = np.ascontiguousarray(samples, np.float32)
        l1, l2, fl = C.c_double(), C.c_double(), C.c_double()
        self.lib.orc_final_loss(C.byref(m), _fp(X), _fp(y), _fp(samples), C.c_int(samples.shape[0]),
                                C.byref(l1), C.byref(l2), C.byref(fl))
        return l1.value, l2.value, fl.value

    def bench_grad_evals(self, m, X, y, threads, seconds):
        X = np.ascontiguousarray(X, np.float32)
        y = np.ascontiguousarray(y, np.float32)
        used = C.c_int()
        done = C.c_long()
        rate = self.lib.orc_bench_grad_evals(C.byref(m), _fp(X), _fp(y), C.c_int(threads),
                                             C.c_double(seconds), C.byref(used), C.byref(done))
        return rate, used.value, done.value


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "-s"], check=True)


def load():
    if not os.path.exists(LIB):
        build()
    return Oracle(C.CDLL(LIB))
