/*
 * bnn_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the HMC / 2-layer-MLP math of NVIDIA/mcmc-bnn-example, used as the checker for
 * the HIP library.  Nothing under oracle/ is part of the product: only tests/, the smoke check and
 * the cpu_baseline leg of bench.py may load it.  The product never calls into it.
 *
 * Reference files restated (paths relative to the reference checkout):
 *   include/mcmc/mcmc_step_ffma.h   parameter layout 35-44, leapfrog update 106-120, block-0
 *                                   bookkeeping 122-152, forward 225-281, loss/grad 283-310,
 *                                   backward 315-360, tail masking 84-91/102/301, sequencing 395-427
 *   include/mcmc/kernel_helpers.h   tanh 29-44, log-accept 153-188, loss sums 190-216
 *   include/mcmc/main.h             state 48-76, bootstrap 191-202, loop 204-287, accept 235-265,
 *                                   adaptation 267-276, sample store 277-283, final loss 78-115
 *   include/mcmc/global_params.h    all constants
 *
 * Pinning status (what independent evidence each function is checked against in tests/):
 *   orc_philox4x32_10         Random123 known-answer vectors                             pinned
 *   orc_det_log / orc_ppnd16  numpy.log / scipy.special.ndtri                            pinned
 *   orc_normal / orc_uniform  KS test + moments against scipy.stats                      pinned
 *   orc_tanh_fwd/bwd          numpy.tanh in double; identity branch; 1-tanh^2            pinned
 *   orc_row_loglik            scipy.stats.t.logpdf / norm.logpdf; finite differences     pinned
 *   orc_prior_terms           scipy.stats.norm.logpdf                                    pinned
 *   orc_eval_f32 / _f64       numpy float64 forward, torch.autograd gradient, finite
 *                             differences, w = 0 closed form                             pinned
 *   orc_mcmc_step             closed-form harmonic oscillator, textbook leapfrog,
 *                             time reversibility, O(eps^2) energy error                  pinned
 *   orc_log_acpt              H_prev - H_new recomputed from scratch in float64          pinned
 *   orc_accept / orc_adapt    exhaustive small table; closed-form eps product            pinned
 *   orc_run_chain             composition of the above + sample-store invariants         pinned
 *   orc_run_chain_from        equals the tail of orc_run_chain from its own saved state  pinned
 *   row-parallel evaluation   same bits with 1, 3 and 8 threads                          pinned
 *   cut-short trajectories    same decisions / step sizes as full-length NaN ones        pinned
 *   bit-level outputs of the reference's CUDA kernels (atomic order, ex2.approx / rcp.approx ulps,
 *   cub reduction trees, thrust/libstdc++ RNG streams): the reference ships no test vectors and
 *   cannot be built here                                                        parity unpinned
 */
#ifndef BNN_ORACLE_H
#define BNN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_LIK_STUDENT_T = 0, ORC_LIK_GAUSSIAN = 1 };

/* RNG stream ids of the build-defined counter-based generator */
enum { ORC_STREAM_X = 0, ORC_STREAM_TEACHER = 1, ORC_STREAM_NOISE = 2, ORC_STREAM_MOMENTUM = 3,
       ORC_STREAM_ACCEPT = 4 };

typedef struct orc_model {
  int d0;             /* input features (22)            global_params.h:56 */
  int d1;             /* hidden units (40)              global_params.h:56 */
  int n;              /* rows in the full batch (58368) global_params.h:61 */
  int lik_kind;       /* ORC_LIK_*                                          */
  double lik_scale;   /* Student-t scale (100) / Gaussian sigma   global_params.h:39 */
  double lik_df;      /* Student-t degrees of freedom (2.2)       global_params.h:40 */
  double prior_scale; /* Gaussian prior scale (200)               global_params.h:48 */
} orc_model;

typedef struct orc_hmc {
  int leapfrog_steps;   /* 1000  global_params.h:30 */
  int burn_in;          /* 100   global_params.h:28 */
  int n_samples;        /* 800   global_params.h:29 */
  int adapt_steps;      /* = burn_in  global_params.h:36 */
  float eps0;           /* 0.01  global_params.h:32 */
  float target_rate;    /* 0.2   global_params.h:33 */
  float decrement;      /* 0.1   global_params.h:34 */
  float increment;      /* 0.01  global_params.h:35 */
  uint32_t seed;        /* RNG key word 0 */
  uint32_t chain_id;    /* RNG key word 1 (window * chains_per_window + chain) */
} orc_hmc;

int orc_num_params(int d0, int d1);
/* number of OpenMP threads the row-parallel evaluations use from now on (results do not depend on it) */
void orc_set_threads(int threads);
/* 0: orc_mcmc_step integrates every step even after the position has become non-finite (as the
 * reference does); 1 (default): it stops there.  Decisions and step sizes are the same either way;
 * the switch exists so that a test can show it. */
void orc_set_cut_short(int on);

/* ---- RNG (build-defined; replaces main.h:207-216 and main.h:235-239) ---- */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
double orc_det_log(double x);
double orc_det_sqrt(double x);
double orc_ppnd16(double p);
/* word `index` of stream (`stream`, `t`) under key (seed, id) */
uint32_t orc_rng_word(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index);
float orc_normal(uint32_t seed, uint32_t id, uint32_t stream, uint32_t t, uint64_t index);
/* momentum of transition t: out[p] ~ N(0,1), p < P                         (main.h:207-216) */
void orc_momentum(uint32_t seed, uint32_t chain_id, uint32_t t, int P, float* out);
/* log of the accept uniform of transition t, as float                      (main.h:235-239) */
float orc_log_uniform(uint32_t seed, uint32_t chain_id, uint32_t t);

/* ---- synthetic data of the benchmark configs (build-defined generator) ---- */
void orc_gen_window(uint32_t seed, uint32_t window, int n, int d0, int d1, float teacher_scale,
                    float noise_sigma, float* X, float* y, float* teacher /* P or NULL */);

/* ---- scalar pieces ---- */
float orc_tanh_fwd(float x);                      /* kernel_helpers.h:34-42 */
float orc_tanh_bwd(float out, float dgrad);       /* kernel_helpers.h:43    */
/* per-row log-likelihood and d loglik / d yhat given the residual inputs   (ffma.h:289-301) */
void orc_row_loglik(const orc_model* m, float y, float yhat, float b2, float* ell, float* g);
/* per-parameter log-prior and its gradient                                 (ffma.h:114-118) */
void orc_prior_terms(const orc_model* m, float w, float* logp, float* grad);

/* ---- log-posterior and gradient at w ---- */
/* FP32 per-row arithmetic as in ffma.h:225-360; cross-row sums accumulated in double and rounded
 * once.  ell[n], prior[P], grad[P] (likelihood + prior).  yhat may be NULL. */
void orc_eval_f32(const orc_model* m, const float* X, const float* y, const float* w, float* ell,
                  float* prior, float* grad, float* yhat);
/* everything in double with the exact tanh: ground truth for tolerances */
void orc_eval_f64(const orc_model* m, const float* X, const float* y, const double* w, double* ell,
                  double* prior, double* grad);

/* ---- the step operator: L fused leapfrog steps                           (ffma.h:395-427) ----
 * in : w_prev, mom_prev, grad_prev (= full gradient at w_prev), eps, L >= 1
 * out: w_next, mom_next (lacking the final half step), grad_cur (full gradient at w_next),
 *      loss_values[n + P] (per-row log-lik then per-parameter log-prior at w_next)
 * A trajectory whose position leaves the finite numbers is cut short there and returns NaN in every
 * output (the transition would reject whatever the remaining steps did). */
void orc_mcmc_step(const orc_model* m, const float* X, const float* y, const float* w_prev,
                   const float* mom_prev, const float* grad_prev, float eps, int L, float* w_next,
                   float* mom_next, float* grad_cur, float* loss_values);

/* ---- log accept ratio                                                    (kernel_helpers.h:153-188) */
float orc_log_acpt(int n_loss /* n + P */, int P, const float* prev_loss, const float* new_loss,
                   const float* prev_mom, const float* new_mom, const float* grad_cur, float eps);
/* accept rule main.h:242: 1 iff log_u < log_acpt (NaN rejects) */
int orc_accept(float log_u, float log_acpt);
/* step-size update main.h:267-276 (non-finite log_acpt counts as minus infinity) */
float orc_adapt_eps(const orc_hmc* h, float eps, float log_acpt);

/* ---- whole chain: main.h:117-293 with the build's RNG ----
 * samples[n_samples][P]; per-transition traces of length burn_in + n_samples (may be NULL).
 * Returns the number of accepted transitions. */
int orc_run_chain(const orc_model* m, const orc_hmc* h, const float* X, const float* y,
                  float* samples, float* log_acpt_trace, int* accept_trace, float* eps_trace,
                  float* final_w, float* final_eps);

/* The same from a given state: position w0 (P floats, NULL = zeros), step size eps0, first
 * transition index t0 (selects the RNG counters, the adaptation window and the sample slots), for
 * n_trans transitions.  Traces have length n_trans; samples[h->n_samples][P] receives the rows whose
 * transition index falls in [burn_in, burn_in + n_samples). */
int orc_run_chain_from(const orc_model* m, const orc_hmc* h, const float* X, const float* y,
                       const float* w0, float eps0, int t0, int n_trans, float* samples,
                       float* log_acpt_trace, int* accept_trace, float* eps_trace, float* final_w,
                       float* final_eps);

/* mean log-lik / log-prior over samples                                    (main.h:78-115) */
void orc_final_loss(const orc_model* m, const float* X, const float* y, const float* samples,
                    int n_samples, double* loss1, double* loss2, double* full);

/* ---- CPU baseline: gradient evaluations per second with `threads` OpenMP threads, each thread
 * running leapfrog steps on its own window copy for about `seconds`.  Returns evals/s. */
double orc_bench_grad_evals(const orc_model* m, const float* X, const float* y, int threads,
                            double seconds, int* threads_used, long* evals_done);

#ifdef __cplusplus
}
#endif
#endif
